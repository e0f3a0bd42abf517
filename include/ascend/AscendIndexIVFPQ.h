// faiss::ascend::AscendIndexIVFPQ : AscendIndexIVF : AscendIndex : faiss::Index
//   (FR/ascend/AscendIndexIVFPQ.h:32-96, FR/ascend/AscendIndexIVF.h:75-118, FR/ascend/AscendIndex.h:62-110).
// Header-only; every method forwards to the C ABI (include/indexsdk_amd.h).
#pragma once
#include <algorithm>
#include <cstring>

#include "AscendIndexIVF.h"

namespace faiss {
namespace ascend {

// AscendIndexIVFPQConfig (FR/ascend/AscendIndexIVFPQ.h:32-68)
struct AscendIndexIVFPQConfig : public AscendIndexIVFConfig {
    inline AscendIndexIVFPQConfig() : AscendIndexIVFConfig({0}, IVF_DEFAULT_MEM) {}
    explicit inline AscendIndexIVFPQConfig(std::initializer_list<int> devices, int64_t resourceSize = IVF_DEFAULT_MEM)
        : AscendIndexIVFConfig(devices, resourceSize)
    {
    }
    explicit inline AscendIndexIVFPQConfig(std::vector<int> devices, int64_t resourceSize = IVF_DEFAULT_MEM)
        : AscendIndexIVFConfig(std::move(devices), resourceSize)
    {
    }
    int trainSamplesPerList = 40;
    int maxTrainSamples = 10000000;
    int pqNiter = -1;                        // -1: cp.niter
    bool useDistributedCoarse = false;       // no counterpart on one GPU
    bool enableQueryParallelSearch = false;  // no counterpart on one GPU
    // additions of this build
    bool lutFp16 = false;                // per-query LUT stored as IEEE half (distances within 1e-2)
    bool pqSpherical = false;            // sub-quantizer codewords L2-normalised after every update, as the reference's
                                         // host training (useKmeansPP = false) does; its device training does not
    bool strictReferenceParams = false;  // true: enforce the reference's whitelists (dims 128, nlist 1024..16384 /
                                         // 262144 / 524288, msubs 2..32) with its "Unsupported ..." messages
};

class AscendIndexIVFPQ : public AscendIndexIVF {
public:
    AscendIndexIVFPQ(int dims, faiss::MetricType metric, int nlist, int msubs, int nbits,
                     AscendIndexIVFPQConfig config = AscendIndexIVFPQConfig())
        : AscendIndexIVF(dims, metric, nlist, config), ivfPQConfig(config), msubs_(msubs), nbits_(nbits)
    {
        create(dims, metric, nlist, msubs, nbits);
        is_trained = false;
    }
    virtual ~AscendIndexIVFPQ() {}
    AscendIndexIVFPQ(const AscendIndexIVFPQ &) = delete;
    AscendIndexIVFPQ &operator=(const AscendIndexIVFPQ &) = delete;

    void train(idx_t n, const float *x) override
    {
        ixaThrowIfError(ivfpq_train(h_, n, x));
        is_trained = true;
    }
    using AscendIndexIVF::remove_ids;   // by selector
    void remove_ids(size_t n, const idx_t *ids)
    {
        ixaThrowIfError(ivfpq_remove_ids(h_, (int64_t)n, reinterpret_cast<const int64_t *>(ids), nullptr));
        syncTotal();
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

    // Initialize ourselves from the given CPU index; will overwrite (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:392-425).
    // The reference copies the codes as they are and searches them against the RAW query, which is only right
    // for an index built with by_residual = false: here an index with by_residual = true is refused.
    void copyFrom(const faiss::IndexIVFPQ *index)
    {
        if (index == nullptr) {
            throw FaissException("index is nullptr.");
        }
        if (!index->is_trained) {
            throw FaissException("Source index is not trained");
        }
        if (index->by_residual) {
            throw FaissException("copyFrom: the source index encodes residuals (by_residual = true); this index "
                                 "searches codes of the raw vectors (by_residual = false)");
        }
        if (index->pq.nbits != 8 || index->quantizer == nullptr || index->invlists == nullptr ||
            index->quantizer->ntotal != (idx_t)index->nlist || index->invlists->code_size != index->pq.M) {
            throw FaissException("copyFrom: the source index must have 8-bit codes, a filled coarse quantizer and "
                                 "inverted lists of pq.M bytes per entry");
        }
        const auto *flat = dynamic_cast<const faiss::IndexFlat *>(index->quantizer);
        if (flat == nullptr) {
            throw FaissException("copyFrom: the coarse quantizer must be an IndexFlat");
        }
        // a new device index of the source's shape replaces ours (the reference overwrites d, nlist, metric too)
        ivfpq_index_t *old = h_;
        h_ = nullptr;
        try {
            metric_type = index->metric_type;
            create(index->d, index->metric_type, (int)index->nlist, (int)index->pq.M, 8);
        } catch (...) {
            h_ = old;
            throw;
        }
        ivfpq_destroy(old);
        d = index->d;
        nlist = (int)index->nlist;
        msubs_ = (int)index->pq.M;
        ivfConfig.cp = index->cp;
        ixaThrowIfError(ivfpq_set_trained(h_, flat->get_xb(), index->pq.centroids.data()));
        is_trained = true;
        setNumProbes((int)std::min<size_t>(std::max<size_t>(index->nprobe, 1), index->nlist));
        for (size_t l = 0; l < index->nlist; l++) {
            const size_t n = index->invlists->list_size(l);
            if (n == 0) {
                continue;
            }
            const uint8_t *codes = index->invlists->get_codes(l);
            const idx_t *ids = index->invlists->get_ids(l);
            const int rc = ivfpq_add_codes(h_, (int64_t)l, (int64_t)n, codes, reinterpret_cast<const int64_t *>(ids));
            index->invlists->release_codes(l, codes);
            index->invlists->release_ids(l, ids);
            ixaThrowIfError(rc);
        }
        syncTotal();
    }

    // Copy ourselves to the given CPU index; will overwrite all data (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:453-508)
    void copyTo(faiss::IndexIVFPQ *index) const
    {
        if (index == nullptr) {
            throw FaissException("index is nullptr.");
        }
        if (!is_trained) {
            throw FaissException("Index is not trained");
        }
        if (index->ntotal > 0) {
            index->reset();
        }
        index->d = d;
        index->metric_type = metric_type;
        index->is_trained = true;
        index->nlist = (size_t)nlist;
        index->nprobe = (size_t)getNumProbes();
        index->by_residual = false;
        index->cp = ivfConfig.cp;
        index->pq.d = (size_t)d;
        index->pq.M = (size_t)msubs_;
        index->pq.nbits = 8;
        index->pq.set_derived_values();
        std::vector<float> centroids((size_t)nlist * d);
        ixaThrowIfError(ivfpq_get_trained(h_, centroids.data(), index->pq.centroids.data()));
        faiss::IndexFlat *quantizer = metric_type == faiss::METRIC_INNER_PRODUCT
                                          ? static_cast<faiss::IndexFlat *>(new faiss::IndexFlatIP(d))
                                          : static_cast<faiss::IndexFlat *>(new faiss::IndexFlatL2(d));
        quantizer->add(nlist, centroids.data());
        if (index->own_fields) {
            delete index->quantizer;
        }
        index->quantizer = quantizer;
        index->own_fields = true;
        index->code_size = (size_t)msubs_;
        faiss::InvertedLists *ivf = new faiss::ArrayInvertedLists((size_t)nlist, index->code_size);
        index->replace_invlists(ivf, true);
        std::vector<uint8_t> codes;
        std::vector<ascend_idx_t> ids;
        index->ntotal = 0;
        for (int l = 0; l < nlist; l++) {
            getListCodesAndIds(l, codes, ids);
            if (!ids.empty()) {
                ivf->add_entries((size_t)l, ids.size(), reinterpret_cast<const idx_t *>(ids.data()), codes.data());
                index->ntotal += (idx_t)ids.size();
            }
        }
    }

    // ---- additions of this build -----------------------------------------------------------------------------
    // Quantizer exchange without faiss types: centroids[nlist*d], codebook[msubs*256*(d/msubs)].
    void copyFromTrained(const float *centroids, const float *codebook)
    {
        ixaThrowIfError(ivfpq_set_trained(h_, centroids, codebook));
        is_trained = true;
    }
    void copyToTrained(float *centroids, float *codebook) const
    {
        ixaThrowIfError(ivfpq_get_trained(h_, centroids, codebook));
    }
    // ascend::IndexIVFPQ::addPQCodes (FR/ascenddaemon/impl/IndexIVFPQ.cpp:210-235)
    void addPQCodes(int listId, size_t n, const uint8_t *codes, const idx_t *ids)
    {
        ixaThrowIfError(ivfpq_add_codes(h_, listId, (int64_t)n, codes, reinterpret_cast<const int64_t *>(ids)));
        syncTotal();
    }
    // File form of copyTo / copyFrom: the byte layout of faiss::write_index for an IndexIVFPQ with
    // by_residual = false.  readFaiss replaces this object's index; the file must have the dims, metric,
    // nlist and msubs this object was constructed with.
    void writeFaiss(const char *path) const { ixaThrowIfError(ivfpq_write_faiss(h_, path)); }
    void readFaiss(const char *path)
    {
        ivfpq_index_t *loaded = nullptr;
        ixaThrowIfError(ivfpq_read_faiss(path, nullptr, &loaded));
        int fd = 0, fm = 0, fM = 0;
        int64_t fl = 0;
        ivfpq_get_shape(loaded, &fd, &fm, &fl, &fM);
        if (fd != d || fm != (int)metric_type || fl != nlist || fM != msubs_) {
            ivfpq_destroy(loaded);
            throw FaissException("the file's dims / metric / nlist / msubs differ from this index");
        }
        ivfpq_destroy(h_);
        h_ = loaded;
        is_trained = true;
        syncTotal();
    }

protected:
    void create(int dims, faiss::MetricType metric, int nlist_, int msubs, int nbits)
    {
        ivfpq_config_t c;
        ivfpq_config_default(&c);
        c.niter = ivfPQConfig.cp.niter;
        c.pq_niter = ivfPQConfig.pqNiter;
        c.spherical = ivfPQConfig.cp.spherical ? 1 : -1;   // -1: on for inner product, as the reference forces it
        c.train_samples_per_list = ivfPQConfig.trainSamplesPerList;
        c.max_train_samples = ivfPQConfig.maxTrainSamples;
        c.lut_fp16 = ivfPQConfig.lutFp16 ? 1 : 0;
        c.pq_spherical = ivfPQConfig.pqSpherical ? 1 : 0;
        c.strict_reference_params = ivfPQConfig.strictReferenceParams ? 1 : 0;
        if (ivfPQConfig.resourceSize > c.scratch_bytes) {
            c.scratch_bytes = ivfPQConfig.resourceSize;
        }
        ixaThrowIfError(ivfpq_create(dims, (int)metric, nlist_, msubs, nbits, &c, &h_));
        codeSize = msubs;
    }
    AscendIndexIVFPQConfig ivfPQConfig;
    int msubs_, nbits_;
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
