// faiss::ascend::AscendIndexIVF : AscendIndex   (FR/ascend/AscendIndexIVF.h:37-118): what every inverted-file
// index of the reference offers above AscendIndex.  The one inverted-file family this build serves is IVFPQ,
// so the level works on an ivfpq handle that the derived class creates.
#pragma once
#include "AscendIndex.h"

namespace faiss {
namespace ascend {

const int64_t IVF_DEFAULT_MEM = 0x8000000;   // 128M

// AscendIndexIVFConfig (FR/ascend/AscendIndexIVF.h:37-72)
struct AscendIndexIVFConfig : public AscendIndexConfig {
    inline AscendIndexIVFConfig() : AscendIndexConfig({0}, IVF_DEFAULT_MEM), useKmeansPP(false)
    {
        SetDefaultClusteringConfig();
    }
    inline AscendIndexIVFConfig(std::initializer_list<int> devices, int64_t resourceSize = IVF_DEFAULT_MEM)
        : AscendIndexConfig(devices, resourceSize), useKmeansPP(false)
    {
        SetDefaultClusteringConfig();
    }
    inline AscendIndexIVFConfig(std::vector<int> devices, int64_t resourceSize = IVF_DEFAULT_MEM)
        : AscendIndexConfig(std::move(devices), resourceSize), useKmeansPP(false)
    {
        SetDefaultClusteringConfig();
    }
    inline void SetDefaultClusteringConfig()
    {
        // a low number of iterations: this is typically used for large clusterings
        cp.niter = 10;
    }
    // configuration of the coarse quantizer object (no separate object exists here; kept for source compatibility)
    AscendIndexConfig flatConfig;
    // The reference trains on the NPU when set and with faiss::Clustering on the host otherwise.  This build
    // always trains on the device (Lloyd iterations seeded with random samples): the flag is accepted and
    // changes nothing.
    bool useKmeansPP;
    // clustering parameters of the coarse quantizer: cp.niter and cp.spherical are honoured (spherical is also
    // switched on for inner product, as the reference does); the other fields have no counterpart.
    ClusteringParameters cp;
};

class AscendIndexIVF : public AscendIndex {
public:
    virtual ~AscendIndexIVF()
    {
        if (h_) {
            ivfpq_destroy(h_);
        }
    }
    AscendIndexIVF(const AscendIndexIVF &) = delete;
    AscendIndexIVF &operator=(const AscendIndexIVF &) = delete;

    // number of inverted lists
    int getNumLists() const { return nlist; }
    // clears all inverted lists, keeps the trained quantizers
    void reset() override
    {
        ixaThrowIfError(ivfpq_reset(h_));
        syncTotal();
    }
    virtual void setNumProbes(int nprobes) { ixaThrowIfError(ivfpq_set_nprobe(h_, nprobes)); }
    int getNumProbes() const
    {
        int v = 0;
        ixaThrowIfError(ivfpq_get_nprobe(h_, &v));
        return v;
    }
    void reserveMemory(size_t numVecs) override { ixaThrowIfError(ivfpq_reserve_memory(h_, (int64_t)numVecs)); }
    size_t reclaimMemory() override
    {
        int64_t bytes = 0;
        ixaThrowIfError(ivfpq_reclaim_memory(h_, &bytes));
        return (size_t)bytes;
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
        codes.resize((size_t)len * codeSize);
        ids.resize(len);
        ixaThrowIfError(ivfpq_get_list(h_, listId, codes.data(), reinterpret_cast<int64_t *>(ids.data())));
    }
    // remove_ids(const IDSelector &) (FR/ascend/AscendIndex.h:78 -> AscendIndexIVFImpl::removeImpl,
    // FR/ascend/impl/AscendIndexIVFImpl.cpp:413-460): a batch or a range of ids; lists keep their order.  A
    // selector of another kind (the reference ignores it) is asked about every stored id.
    size_t remove_ids(const faiss::IDSelector &sel) override
    {
        std::vector<int64_t> ids;
        int64_t imin = 0, imax = 0, removed = 0;
        auto allIds = [this](std::vector<idx_t> &m) {
            m.clear();
            std::vector<uint8_t> codes;
            std::vector<ascend_idx_t> listIds;
            for (int l = 0; l < nlist; l++) {
                getListCodesAndIds(l, codes, listIds);
                m.insert(m.end(), listIds.begin(), listIds.end());
            }
        };
        if (ixaSelectorIds(sel, allIds, ids, imin, imax)) {
            ixaThrowIfError(ivfpq_remove_range(h_, imin, imax, &removed));
        } else {
            ixaThrowIfError(ivfpq_remove_ids(h_, (int64_t)ids.size(), ids.data(), &removed));
        }
        syncTotal();
        return (size_t)removed;
    }
    using AscendIndex::add;            // the IEEE half overloads
    using AscendIndex::add_with_ids;
    using AscendIndex::search;
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
    ivfpq_index_t *handle() const { return h_; }

protected:
    AscendIndexIVF(int dims, faiss::MetricType metric, int nlist_, AscendIndexIVFConfig config)
        : AscendIndex(dims, metric, config), nlist(nlist_), ivfConfig(std::move(config))
    {
    }
    void syncTotal()
    {
        int64_t v = 0;
        ixaThrowIfError(ivfpq_ntotal(h_, &v));
        ntotal = v;
    }
    int nlist;
    int codeSize = 0;           // bytes per code of a list entry
    AscendIndexIVFConfig ivfConfig;
    ivfpq_index_t *h_ = nullptr;
};

}  // namespace ascend
}  // namespace faiss
