// Cloning between CPU (faiss) indexes and the device indexes of this library, with the reference's entry
// points and options (FR/ascend/AscendCloner.h:34-47, FR/ascend/AscendClonerOptions.h:24-40):
//   index_ascend_to_cpu:  AscendIndexFlat    -> IndexIDMap over IndexFlat (FR/ascend/AscendCloner.cpp:64-70)
//                         AscendIndexIVFPQ   -> IndexIVFPQ with by_residual = false (copyTo)
//   index_cpu_to_ascend:  IndexFlat, IndexIDMap over IndexFlat -> AscendIndexFlat (FR/ascend/AscendCloner.cpp:133-165)
//                         IndexIVFPQ (by_residual = false)     -> AscendIndexIVFPQ (copyFrom)
//   index_int8_ascend_to_cpu / index_int8_cpu_to_ascend: AscendIndexInt8Flat <-> IndexIDMap over
//                         IndexScalarQuantizer (one int8 per dimension in its codes)
// The reference's cloner does not know its IVFPQ index; the two IVFPQ directions are this build's addition, on
// top of the copyFrom / copyTo the reference does have.  The caller owns what is returned.  Header-only.
#pragma once
#include <initializer_list>
#include <memory>
#include <vector>

#include "AscendIndexFlat.h"
#include "AscendIndexIVFPQ.h"

namespace faiss {
namespace ascend {

struct AscendClonerOptions {
    long reserveVecs = 0;
    bool verbose = false;
    int64_t resourceSize = IVF_DEFAULT_MEM;
    bool slim = false;         // scalar-quantizer indexes only: accepted for source compatibility
    bool filterable = false;
    uint32_t indexMode = 0;
    uint32_t blockSize = DEFAULT_BLOCK_SIZE;
};

inline faiss::Index *index_ascend_to_cpu(const faiss::Index *ascend_index)
{
    if (auto flat = dynamic_cast<const AscendIndexFlat *>(ascend_index)) {
        std::unique_ptr<faiss::IndexFlat> rows(new faiss::IndexFlat(flat->d, flat->metric_type));
        std::unique_ptr<faiss::IndexIDMap> res(new faiss::IndexIDMap(rows.get()));
        res->own_fields = true;
        rows.release();
        flat->copyTo(res.get());
        return res.release();
    }
    if (auto ivfpq = dynamic_cast<const AscendIndexIVFPQ *>(ascend_index)) {
        std::unique_ptr<faiss::IndexIVFPQ> res(new faiss::IndexIVFPQ());
        ivfpq->copyTo(res.get());
        return res.release();
    }
    throw faiss::FaissException("clone from ascend to cpu not supported for this type of Index");
}

inline faiss::Index *index_cpu_to_ascend(std::vector<int> devices, const faiss::Index *index,
                                         const AscendClonerOptions *options = nullptr)
{
    if (devices.empty()) {
        throw faiss::FaissException("device list can not be empty!");
    }
    const AscendClonerOptions opt = options ? *options : AscendClonerOptions();
    if (auto flat = dynamic_cast<const faiss::IndexFlat *>(index)) {
        return new AscendIndexFlat(flat, AscendIndexFlatConfig(devices, opt.resourceSize));
    }
    if (auto idm = dynamic_cast<const faiss::IndexIDMap *>(index)) {
        if (dynamic_cast<const faiss::IndexFlat *>(idm->index)) {
            return new AscendIndexFlat(idm, AscendIndexFlatConfig(devices, opt.resourceSize));
        }
    }
    if (auto ivfpq = dynamic_cast<const faiss::IndexIVFPQ *>(index)) {
        std::unique_ptr<AscendIndexIVFPQ> res(new AscendIndexIVFPQ(ivfpq->d, ivfpq->metric_type, (int)ivfpq->nlist,
                                                                   (int)ivfpq->pq.M, (int)ivfpq->pq.nbits,
                                                                   AscendIndexIVFPQConfig(devices, opt.resourceSize)));
        res->copyFrom(ivfpq);
        if (opt.reserveVecs > 0) {
            res->reserveMemory((size_t)opt.reserveVecs);
        }
        return res.release();
    }
    throw faiss::FaissException("clone from cpu to ascend not supported for this type of Index");
}

inline faiss::Index *index_cpu_to_ascend(std::initializer_list<int> devices, const faiss::Index *index,
                                         const AscendClonerOptions *options = nullptr)
{
    return index_cpu_to_ascend(std::vector<int>(devices), index, options);
}

// int8 indexes (FR/ascend/AscendCloner.h:42-47; FR/ascend/AscendCloner.cpp:97-113, 205-230): AscendIndexInt8Flat
// <-> IndexIDMap over an IndexScalarQuantizer whose codes are the int8 vectors
inline faiss::Index *index_int8_ascend_to_cpu(const AscendIndexInt8 *index)
{
    if (auto flat = dynamic_cast<const AscendIndexInt8Flat *>(index)) {
        std::unique_ptr<faiss::IndexScalarQuantizer> codes(new faiss::IndexScalarQuantizer());
        std::unique_ptr<faiss::IndexIDMap> res(new faiss::IndexIDMap(codes.get()));
        res->own_fields = true;
        codes.release();
        flat->copyTo(res.get());
        return res.release();
    }
    throw faiss::FaissException("clone from ascend to cpu not supported for this type of Index");
}

inline AscendIndexInt8 *index_int8_cpu_to_ascend(std::vector<int> devices, const faiss::Index *index,
                                                 const AscendClonerOptions *options = nullptr)
{
    if (devices.empty()) {
        throw faiss::FaissException("device list can not be empty!");
    }
    const AscendClonerOptions opt = options ? *options : AscendClonerOptions();
    AscendIndexInt8FlatConfig config;
    config.deviceList = devices;
    config.resourceSize = opt.resourceSize;
    if (auto sq = dynamic_cast<const faiss::IndexScalarQuantizer *>(index)) {
        return new AscendIndexInt8Flat(sq, config);
    }
    if (auto idm = dynamic_cast<const faiss::IndexIDMap *>(index)) {
        if (dynamic_cast<const faiss::IndexScalarQuantizer *>(idm->index)) {
            return new AscendIndexInt8Flat(idm, config);
        }
    }
    throw faiss::FaissException("clone from cpu to ascend not supported for this type of Index");
}

inline AscendIndexInt8 *index_int8_cpu_to_ascend(std::initializer_list<int> devices, const faiss::Index *index,
                                                 const AscendClonerOptions *options = nullptr)
{
    return index_int8_cpu_to_ascend(std::vector<int>(devices), index, options);
}

}  // namespace ascend
}  // namespace faiss
