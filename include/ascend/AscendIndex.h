// Header-only C++ face of the MI355X search path with the reference's class shape, root of the hierarchy:
//   faiss::ascend::AscendIndex : faiss::Index      (FR/ascend/AscendIndex.h:41-110)
// Every method of the classes built on it forwards to the C ABI (include/indexsdk_amd.h) and throws
// faiss::FaissException on a non-zero status, as the reference's public layer does (FAISS_THROW_IF_NOT_FMT).
#pragma once
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <string>
#include <vector>

#include "../faiss_shim.h"
#include "../indexsdk_amd.h"

namespace faiss {
namespace ascend {

using ascend_idx_t = uint64_t;  // FR/ascend/AscendIndex.h:45

const idx_t MAX_N = 1000000000;
const idx_t MAX_K = 4096;
const int64_t INDEX_DEFAULT_MEM = 0x2000000;   // 32M
const uint32_t DEFAULT_BLOCK_SIZE = 16384 * 16;

// IEEE binary16 -> binary32, exact (subnormals, infinities and NaNs included).
inline float ixaHalfToFloat(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                shift++;
            }
            bits = sign | ((uint32_t)(113 - shift) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline void ixaThrowIfError(int status)
{
    if (status != IXA_OK) {
        throw faiss::FaissException(ixa_last_error());
    }
}

// AscendIndexConfig (FR/ascend/AscendIndex.h:51-71).  deviceList is accepted for source compatibility: this
// build serves exactly one GPU, the current HIP device.  resourceSize bounds the scratch of a search
// (raised to this build's minimum where smaller).
struct AscendIndexConfig {
    inline AscendIndexConfig() : deviceList({0}), resourceSize(INDEX_DEFAULT_MEM), dBlockSize(DEFAULT_BLOCK_SIZE) {}
    inline AscendIndexConfig(std::initializer_list<int> devices, int64_t resources = INDEX_DEFAULT_MEM,
                             uint32_t blockSize = DEFAULT_BLOCK_SIZE)
        : deviceList(devices), resourceSize(resources), dBlockSize(blockSize)
    {
    }
    inline AscendIndexConfig(std::vector<int> devices, int64_t resources = INDEX_DEFAULT_MEM,
                             uint32_t blockSize = DEFAULT_BLOCK_SIZE)
        : deviceList(std::move(devices)), resourceSize(resources), dBlockSize(blockSize)
    {
    }
    std::vector<int> deviceList;
    int64_t resourceSize;
    bool slim = false;
    bool filterable = false;
    uint32_t dBlockSize = DEFAULT_BLOCK_SIZE;
};

class AscendIndex : public faiss::Index {
public:
    AscendIndex(int dims, faiss::MetricType metric, AscendIndexConfig config)
        : faiss::Index(dims, metric), indexConfig(std::move(config))
    {
    }
    virtual ~AscendIndex() {}
    AscendIndex(const AscendIndex &) = delete;
    AscendIndex &operator=(const AscendIndex &) = delete;

    // reserve memory for the database (FR/ascend/AscendIndex.h:91-92); a family without growable storage ignores it
    virtual void reserveMemory(size_t /*numVecs*/) {}
    // reclaim device memory to exactly the amount needed; returns the bytes released (:94-96)
    virtual size_t reclaimMemory() { return 0; }
    std::vector<int> getDeviceList() { return indexConfig.deviceList; }

    // The reference's calls with IEEE half inputs (FR/ascend/AscendIndex.h:103-107).  Its indexes store and
    // compare in half precision anyway; this build computes in fp32, so the halves are widened (exactly) first.
    void add(idx_t n, const uint16_t *x) { add_with_ids(n, x, nullptr); }
    void add_with_ids(idx_t n, const uint16_t *x, const idx_t *ids)
    {
        const std::vector<float> wide = ixaWiden(n, x);
        if (ids) {
            add_with_ids(n, wide.data(), ids);
        } else {
            add(n, wide.data());
        }
    }
    void search(idx_t n, const uint16_t *x, idx_t k, float *distances, idx_t *labels) const
    {
        const std::vector<float> wide = ixaWiden(n, x);
        search(n, wide.data(), k, distances, labels);
    }
    using faiss::Index::add;
    using faiss::Index::add_with_ids;
    using faiss::Index::search;

protected:
    std::vector<float> ixaWiden(idx_t n, const uint16_t *x) const
    {
        if (x == nullptr || n < 0) {
            throw faiss::FaissException("x can not be nullptr.");
        }
        std::vector<float> out((size_t)n * d);
        for (size_t i = 0; i < out.size(); i++) {
            out[i] = ixaHalfToFloat(x[i]);
        }
        return out;
    }
    AscendIndexConfig indexConfig;
};

// The ids a selector names, for the C ABI's remove calls: a range stays a range (isRange), a batch or an
// array is listed from its own members, any other selector is asked about every id of `idMap` (the index's
// ids in storage order, fetched by `fetchIdMap` only in that case).
template <typename FetchIdMap>
inline bool ixaSelectorIds(const faiss::IDSelector &sel, FetchIdMap fetchIdMap, std::vector<int64_t> &ids, int64_t &imin,
                           int64_t &imax)
{
    if (auto range = dynamic_cast<const faiss::IDSelectorRange *>(&sel)) {
        imin = range->imin;
        imax = range->imax;
        return true;
    }
    ids.clear();
    if (auto batch = dynamic_cast<const faiss::IDSelectorBatch *>(&sel)) {
        ids.assign(batch->set.begin(), batch->set.end());
    } else if (auto array = dynamic_cast<const faiss::IDSelectorArray *>(&sel)) {
        ids.assign(array->ids, array->ids + array->n);
    } else {
        std::vector<faiss::idx_t> idMap;
        fetchIdMap(idMap);
        for (faiss::idx_t id : idMap) {
            if (sel.is_member(id)) {
                ids.push_back(id);
            }
        }
    }
    return false;
}

}  // namespace ascend
}  // namespace faiss
