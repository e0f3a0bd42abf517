// Header-only C++ face of the MI355X IVFPQ path with the reference's class shape:
//   faiss::ascend::AscendIndexIVFPQ : AscendIndexIVF : AscendIndex : faiss::Index
//   (FR/ascend/AscendIndexIVFPQ.h:71-96, FR/ascend/AscendIndexIVF.h:75-118, FR/ascend/AscendIndex.h:62-110).
// Every method forwards to the C ABI (include/indexsdk_amd.h) and throws faiss::FaissException on
// a non-zero status, as the reference's public layer does (FAISS_THROW_IF_NOT_FMT).
#pragma once
#include <cstdint>
#include <initializer_list>
#include <string>
#include <vector>

#include "../faiss_shim.h"
#include "../indexsdk_amd.h"

namespace faiss {
namespace ascend {

using ascend_idx_t = uint64_t;  // FR/ascend/utils/AscendUtils.h

inline void ixaThrowIfError(int status)
{
    if (status != IXA_OK) {
        throw faiss::FaissException(ixa_last_error());
    }
}

const int64_t IVF_DEFAULT_MEM = 0x8000000;

// AscendIndexIVFPQConfig (FR/ascend/AscendIndexIVFPQ.h:32-68).  deviceList is accepted for source
// compatibility; this build serves exactly one GPU and uses the current HIP device.
struct AscendIndexIVFPQConfig {
    AscendIndexIVFPQConfig() : deviceList({0}), resourceSize(IVF_DEFAULT_MEM) {}
    explicit AscendIndexIVFPQConfig(std::initializer_list<int> devices, int64_t resources = IVF_DEFAULT_MEM)
        : deviceList(devices), resourceSize(resources)
    {
    }
    explicit AscendIndexIVFPQConfig(std::vector<int> devices, int64_t resources = IVF_DEFAULT_MEM)
        : deviceList(std::move(devices)), resourceSize(resources)
    {
    }
    std::vector<int> deviceList;
    int64_t resourceSize;
    bool useKmeansPP = false;
    int trainSamplesPerList = 40;
    int maxTrainSamples = 10000000;
    int pqNiter = -1;
    bool useDistributedCoarse = false;       // no counterpart on one GPU
    bool enableQueryParallelSearch = false;  // no counterpart on one GPU
    // additions of this build
    int niter = 25;               // coarse k-means iterations (the reference's CPU mode uses 25)
    bool spherical = false;       // the reference trains spherical k-means; plain Lloyd is the default here
    bool lutFp16 = false;         // per-query LUT stored as IEEE half
    bool strictReferenceParams = true;  // enforce the reference's d / nlist / msubs whitelists
};

class AscendIndexIVFPQ : public faiss::Index {
public:
    AscendIndexIVFPQ(int dims, faiss::MetricType metric, int nlist, int msubs, int nbits,
                     AscendIndexIVFPQConfig config = AscendIndexIVFPQConfig())
        : faiss::Index(dims, metric), nlist_(nlist), msubs_(msubs)
    {
        ivfpq_config_t c;
        ivfpq_config_default(&c);
        c.niter = config.niter;
        c.pq_niter = config.pqNiter;
        c.spherical = config.spherical ? 1 : 0;
        c.train_samples_per_list = config.trainSamplesPerList;
        c.max_train_samples = config.maxTrainSamples;
        c.lut_fp16 = config.lutFp16 ? 1 : 0;
        c.strict_reference_params = config.strictReferenceParams ? 1 : 0;
        if (config.resourceSize > c.scratch_bytes) {
            c.scratch_bytes = config.resourceSize;
        }
        ixaThrowIfError(ivfpq_create(dims, (int)metric, nlist, msubs, nbits, &c, &h_));
        is_trained = false;
    }
    virtual ~AscendIndexIVFPQ() { ivfpq_destroy(h_); }
    AscendIndexIVFPQ(const AscendIndexIVFPQ &) = delete;
    AscendIndexIVFPQ &operator=(const AscendIndexIVFPQ &) = delete;

    void train(idx_t n, const float *x) override
    {
        ixaThrowIfError(ivfpq_train(h_, n, x));
        is_trained = true;
    }
    void add(idx_t n, const float *x) override { add_with_ids(n, x, nullptr); }
    void add_with_ids(idx_t n, const float *x, const idx_t *ids) override
    {
        ixaThrowIfError(ivfpq_add_with_ids(h_, n, x, reinterpret_cast<const int64_t *>(ids)));
        syncTotal();
    }
    void search(idx_t n, const float *x, idx_t k, float *distances, idx_t *labels,
                const SearchParameters * = nullptr) const override
    {
        ixaThrowIfError(ivfpq_search(h_, n, x, k, distances, reinterpret_cast<int64_t *>(labels)));
    }
    void reset() override
    {
        ixaThrowIfError(ivfpq_reset(h_));
        syncTotal();
    }
    size_t remove_ids(size_t n, const idx_t *ids)
    {
        int64_t removed = 0;
        ixaThrowIfError(ivfpq_remove_ids(h_, (int64_t)n, reinterpret_cast<const int64_t *>(ids), &removed));
        syncTotal();
        return (size_t)removed;
    }
    std::vector<idx_t> update(idx_t n, const float *x, const idx_t *ids)
    {
        std::vector<idx_t> missing((size_t)n);
        int64_t nm = 0;
        ixaThrowIfError(ivfpq_update(h_, n, x, reinterpret_cast<const int64_t *>(ids),
                                     reinterpret_cast<int64_t *>(missing.data()), &nm));
        missing.resize((size_t)nm);
        syncTotal();
        return missing;
    }
    // AscendIndexIVF
    int getNumLists() const { return nlist_; }
    virtual void setNumProbes(int nprobes) { ixaThrowIfError(ivfpq_set_nprobe(h_, nprobes)); }
    int getNumProbes() const
    {
        int v = 0;
        ixaThrowIfError(ivfpq_get_nprobe(h_, &v));
        return v;
    }
    virtual uint32_t getListLength(int listId) const
    {
        int64_t v = 0;
        ixaThrowIfError(ivfpq_list_length(h_, listId, &v));
        return (uint32_t)v;
    }
    virtual void getListCodesAndIds(int listId, std::vector<uint8_t> &codes, std::vector<ascend_idx_t> &ids) const
    {
        const uint32_t len = getListLength(listId);
        codes.resize((size_t)len * msubs_);
        ids.resize(len);
        ixaThrowIfError(ivfpq_get_list(h_, listId, codes.data(), reinterpret_cast<int64_t *>(ids.data())));
    }
    // Quantizer exchange: the part of copyFrom / copyTo (faiss::IndexIVFPQ with by_residual = false)
    // that does not need faiss types.  centroids[nlist*d], codebook[msubs*256*(d/msubs)].
    void copyFromTrained(const float *centroids, const float *codebook)
    {
        ixaThrowIfError(ivfpq_set_trained(h_, centroids, codebook));
        is_trained = true;
    }
    void copyToTrained(float *centroids, float *codebook) const
    {
        ixaThrowIfError(ivfpq_get_trained(h_, centroids, codebook));
    }
    void addPQCodes(int listId, size_t n, const uint8_t *codes, const idx_t *ids)
    {
        ixaThrowIfError(ivfpq_add_codes(h_, listId, (int64_t)n, codes, reinterpret_cast<const int64_t *>(ids)));
        syncTotal();
    }
    // File form of copyTo / copyFrom(faiss::IndexIVFPQ *): the byte layout of faiss::write_index for an
    // IndexIVFPQ with by_residual = false.  readFaiss replaces this object's index; the file must have the
    // dims, metric, nlist and msubs this object was constructed with.
    void writeFaiss(const char *path) const { ixaThrowIfError(ivfpq_write_faiss(h_, path)); }
    void readFaiss(const char *path)
    {
        ivfpq_index_t *loaded = nullptr;
        ixaThrowIfError(ivfpq_read_faiss(path, nullptr, &loaded));
        int fd = 0, fm = 0, fM = 0;
        int64_t fl = 0;
        ivfpq_get_shape(loaded, &fd, &fm, &fl, &fM);
        if (fd != d || fm != (int)metric_type || fl != nlist_ || fM != msubs_) {
            ivfpq_destroy(loaded);
            throw FaissException("the file's dims / metric / nlist / msubs differ from this index");
        }
        ivfpq_destroy(h_);
        h_ = loaded;
        is_trained = true;
        syncTotal();
    }
    ivfpq_index_t *handle() const { return h_; }

protected:
    void syncTotal()
    {
        int64_t v = 0;
        ixaThrowIfError(ivfpq_ntotal(h_, &v));
        ntotal = v;
    }
    ivfpq_index_t *h_ = nullptr;
    int nlist_, msubs_;
};

// AscendIndexImpl::mergeSearchResult (FR/ascend/impl/AscendIndexImpl.cpp:587-640) for callers that
// shard an index over several devices themselves: dist[j] / label[j] hold the [n][k] results of shard j.
inline void mergeSearchResult(const std::vector<std::vector<float>> &dist,
                              const std::vector<std::vector<idx_t>> &label, idx_t n, idx_t k, MetricType metric,
                              float *distances, idx_t *labels)
{
    std::vector<const float *> dp;
    std::vector<const int64_t *> lp;
    for (size_t j = 0; j < dist.size(); j++) {
        dp.push_back(dist[j].data());
        lp.push_back(reinterpret_cast<const int64_t *>(label[j].data()));
    }
    ixaThrowIfError(ixa_merge_search_results((int)dist.size(), n, k, (int)metric, dp.data(), lp.data(), distances,
                                             reinterpret_cast<int64_t *>(labels)));
}

}  // namespace ascend
}  // namespace faiss
