// Header-only C++ faces of the Flat paths with the reference's class shapes:
//   faiss::ascend::AscendIndexFlat : AscendIndex, AscendIndexFlatL2   (FR/ascend/AscendIndexFlat.h:34-110)
//   faiss::ascend::AscendIndexInt8Flat : AscendIndexInt8              (FR/ascend/AscendIndexInt8Flat.h:30-100)
// forwarding to the C ABI (include/indexsdk_amd.h).
#pragma once
#include <cfloat>
#include <vector>

#include "AscendIndex.h"
#include "AscendIndexInt8.h"

namespace faiss {
namespace ascend {

const int64_t FLAT_DEFAULT_MEM = 0x8000000;   // 128M

// The score scratch of a Flat search: the library's default (0) unless the caller's resourceSize asks for more
// (the reference's defaults of 32M / 128M size a different kind of pool).
inline int64_t scratchOf(int64_t resourceSize) { return resourceSize > ((int64_t)1 << 30) ? resourceSize : 0; }

// AscendIndexFlatConfig (FR/ascend/AscendIndexFlat.h:34-45)
struct AscendIndexFlatConfig : public AscendIndexConfig {
    inline AscendIndexFlatConfig() {}
    inline AscendIndexFlatConfig(std::initializer_list<int> devices, int64_t resourceSize = FLAT_DEFAULT_MEM)
        : AscendIndexConfig(devices, resourceSize)
    {
    }
    inline AscendIndexFlatConfig(std::vector<int> devices, int64_t resourceSize = FLAT_DEFAULT_MEM)
        : AscendIndexConfig(std::move(devices), resourceSize)
    {
    }
};

class AscendIndexFlat : public AscendIndex {
public:
    // Construct an empty instance that can be added to
    AscendIndexFlat(int dims, faiss::MetricType metric, AscendIndexFlatConfig config = AscendIndexFlatConfig())
        : AscendIndex(dims, metric, config)
    {
        ixaThrowIfError(flat_create(dims, (int)metric, scratchOf(config.resourceSize), &h_));
    }
    // Construct from a pre-existing faiss::IndexFlat instance
    explicit AscendIndexFlat(const faiss::IndexFlat *index, AscendIndexFlatConfig config = AscendIndexFlatConfig())
        : AscendIndex(index ? index->d : 0, index ? index->metric_type : faiss::METRIC_L2, config)
    {
        if (index == nullptr) {
            throw FaissException("index is nullptr.");
        }
        ixaThrowIfError(flat_create(index->d, (int)index->metric_type, scratchOf(config.resourceSize), &h_));
        copyFrom(index);
    }
    virtual ~AscendIndexFlat() { flat_destroy(h_); }
    AscendIndexFlat(const AscendIndexFlat &) = delete;
    AscendIndexFlat &operator=(const AscendIndexFlat &) = delete;

    // Initialize ourselves from the given CPU index; will overwrite all data in ourselves
    void copyFrom(const faiss::IndexFlat *index)
    {
        if (index == nullptr || index->d != d || index->metric_type != metric_type) {
            throw FaissException("copyFrom: the source index must have this index's dims and metric");
        }
        reset();
        if (index->ntotal > 0) {
            add(index->ntotal, index->get_xb());
        }
    }
    // Copy ourselves to the given CPU index; will overwrite all data in the index instance
    void copyTo(faiss::IndexFlat *index) const
    {
        if (index == nullptr) {
            throw FaissException("index is nullptr.");
        }
        index->reset();
        index->d = d;
        index->metric_type = metric_type;
        std::vector<float> xb((size_t)ntotal * d);
        if (ntotal > 0) {
            ixaThrowIfError(flat_get_base(h_, 0, ntotal, xb.data()));
            index->add(ntotal, xb.data());
        }
    }
    // Initialize ourselves from a CPU index with user ids (FR/ascend/AscendIndexFlat.h:52, 62): its rows must
    // be an IndexFlat
    explicit AscendIndexFlat(const faiss::IndexIDMap *index, AscendIndexFlatConfig config = AscendIndexFlatConfig())
        : AscendIndex(index ? index->d : 0, index ? index->metric_type : faiss::METRIC_L2, config)
    {
        if (index == nullptr) {
            throw FaissException("index is nullptr.");
        }
        ixaThrowIfError(flat_create(index->d, (int)index->metric_type, scratchOf(config.resourceSize), &h_));
        try {
            copyFrom(index);
        } catch (...) {
            flat_destroy(h_);
            throw;
        }
    }
    void copyFrom(const faiss::IndexIDMap *index)
    {
        const faiss::IndexFlat *rows = index ? dynamic_cast<const faiss::IndexFlat *>(index->index) : nullptr;
        if (rows == nullptr || rows->d != d || rows->metric_type != metric_type ||
            (idx_t)index->id_map.size() != rows->ntotal) {
            throw FaissException("copyFrom: the source must be an IndexIDMap over an IndexFlat with this index's "
                                 "dims and metric");
        }
        reset();
        if (rows->ntotal > 0) {
            add_with_ids(rows->ntotal, rows->get_xb(), index->id_map.data());
        }
    }
    void copyTo(faiss::IndexIDMap *index) const
    {
        faiss::IndexFlat *rows = index ? dynamic_cast<faiss::IndexFlat *>(index->index) : nullptr;
        if (rows == nullptr) {
            throw FaissException("copyTo: the target must be an IndexIDMap over an IndexFlat");
        }
        copyTo(rows);
        getIdxMap(0, index->id_map);
        index->d = d;
        index->metric_type = metric_type;
        index->ntotal = ntotal;
    }
    using AscendIndex::add;            // the IEEE half overloads
    using AscendIndex::add_with_ids;
    using AscendIndex::search;
    void add(idx_t n, const float *x) override { add_with_ids(n, x, nullptr); }
    void add_with_ids(idx_t n, const float *x, const idx_t *ids) override
    {
        ixaThrowIfError(flat_add_with_ids(h_, n, x, reinterpret_cast<const int64_t *>(ids)));
        syncTotal();
    }
    void search(idx_t n, const float *x, idx_t k, float *distances, idx_t *labels,
                const SearchParameters * = nullptr) const override
    {
        ixaThrowIfError(flat_search(h_, n, x, k, distances, reinterpret_cast<int64_t *>(labels)));
    }
    // search_with_masks (FR/ascend/AscendIndexFlat.h:78-82): query i may only return the vectors whose bit
    // is set in row i of the mask (n rows of ceil(ntotal / 8) bytes; storage position p = bit p % 8 of byte p / 8)
    void search_with_masks(idx_t n, const float *x, idx_t k, float *distances, idx_t *labels, const void *mask) const
    {
        ixaThrowIfError(flat_search_with_masks(h_, n, x, k, static_cast<const uint8_t *>(mask), distances,
                                               reinterpret_cast<int64_t *>(labels)));
    }
    void search_with_masks(idx_t n, const uint16_t *x, idx_t k, float *distances, idx_t *labels, const void *mask) const
    {
        const std::vector<float> wide = ixaWiden(n, x);
        search_with_masks(n, wide.data(), k, distances, labels, mask);
    }
    void reset() override
    {
        ixaThrowIfError(flat_reset(h_));
        ntotal = 0;
    }
    // Returns the number of vectors we contain
    size_t getBaseSize(int /*deviceId*/ = 0) const { return (size_t)ntotal; }
    // Returns the vectors we contain (the reference hands them out as fp16 bytes; here they are fp32)
    void getBase(int /*deviceId*/, std::vector<float> &xb) const
    {
        xb.resize((size_t)ntotal * d);
        if (ntotal > 0) {
            ixaThrowIfError(flat_get_base(h_, 0, ntotal, xb.data()));
        }
    }
    // Returns the ids of the vectors we contain, in base order
    void getIdxMap(int /*deviceId*/, std::vector<idx_t> &idxMap) const
    {
        idxMap.resize((size_t)ntotal);
        if (ntotal > 0) {
            ixaThrowIfError(flat_get_ids(h_, 0, ntotal, reinterpret_cast<int64_t *>(idxMap.data())));
        }
    }
    // remove_ids (FR/ascend/AscendIndex.h:78): the vectors the selector names leave; every hole, from the
    // highest position down, is refilled with the vector that is last at that moment, as in the reference
    size_t remove_ids(const faiss::IDSelector &sel) override
    {
        std::vector<int64_t> ids;
        int64_t imin = 0, imax = 0, removed = 0;
        if (ixaSelectorIds(sel, [this](std::vector<idx_t> &m) { getIdxMap(0, m); }, ids, imin, imax)) {
            ixaThrowIfError(flat_remove_range(h_, imin, imax, &removed));
        } else {
            ixaThrowIfError(flat_remove_ids(h_, (int64_t)ids.size(), ids.data(), &removed));
        }
        syncTotal();
        return (size_t)removed;
    }

protected:
    void syncTotal()
    {
        int64_t v = 0;
        ixaThrowIfError(flat_ntotal(h_, &v));
        ntotal = v;
    }
    flat_index_t *h_ = nullptr;
};

class AscendIndexFlatL2 : public AscendIndexFlat {
public:
    explicit AscendIndexFlatL2(int dims, AscendIndexFlatConfig config = AscendIndexFlatConfig())
        : AscendIndexFlat(dims, faiss::METRIC_L2, config)
    {
    }
};

const int64_t INT8_FLAT_DEFAULT_MEM = 0x8000000;

// AscendIndexInt8FlatConfig (FR/ascend/AscendIndexInt8Flat.h:30-57); the block size and index mode steer the
// reference's device layout and have no counterpart here.
struct AscendIndexInt8FlatConfig : public AscendIndexInt8Config {
    inline AscendIndexInt8FlatConfig() : AscendIndexInt8Config({0}, INT8_FLAT_DEFAULT_MEM) {}
    inline AscendIndexInt8FlatConfig(std::initializer_list<int> devices, int64_t resourceSize = INT8_FLAT_DEFAULT_MEM)
        : AscendIndexInt8Config(devices, resourceSize)
    {
    }
    inline AscendIndexInt8FlatConfig(std::vector<int> devices, int64_t resourceSize = INT8_FLAT_DEFAULT_MEM)
        : AscendIndexInt8Config(std::move(devices), resourceSize)
    {
    }
    uint32_t dBlockSize = 16384 * 16;
};

// int8 vectors; L2 only.  search() keeps the reference's float signature (exact below 2^24, rounded to
// nearest above; the reference returns a scaled fp16 value); searchInt32() returns the exact int32 distances.
class AscendIndexInt8Flat : public AscendIndexInt8 {
public:
    explicit AscendIndexInt8Flat(int dims, faiss::MetricType metric = faiss::METRIC_L2,
                                 AscendIndexInt8FlatConfig config = AscendIndexInt8FlatConfig())
        : AscendIndexInt8(dims, metric, config)
    {
        ixaThrowIfError(flat_i8_create(dims, (int)metric, scratchOf(config.resourceSize), &h_));
    }
    // Construct from a CPU index that holds int8 codes (FR/ascend/AscendIndexInt8Flat.h:60-66)
    explicit AscendIndexInt8Flat(const faiss::IndexScalarQuantizer *index,
                                 AscendIndexInt8FlatConfig config = AscendIndexInt8FlatConfig())
        : AscendIndexInt8(index ? index->d : 0, index ? index->metric_type : faiss::METRIC_L2, config)
    {
        if (index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        ixaThrowIfError(flat_i8_create(index->d, (int)index->metric_type, scratchOf(config.resourceSize), &h_));
        try {
            copyFrom(index);
        } catch (...) {
            flat_i8_destroy(h_);
            throw;
        }
    }
    explicit AscendIndexInt8Flat(const faiss::IndexIDMap *index,
                                 AscendIndexInt8FlatConfig config = AscendIndexInt8FlatConfig())
        : AscendIndexInt8(index && index->index ? index->index->d : 0,
                          index && index->index ? index->index->metric_type : faiss::METRIC_L2, config)
    {
        if (index == nullptr || index->index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        ixaThrowIfError(flat_i8_create(d, (int)metric_type, scratchOf(config.resourceSize), &h_));
        try {
            copyFrom(index);
        } catch (...) {
            flat_i8_destroy(h_);
            throw;
        }
    }
    virtual ~AscendIndexInt8Flat() { flat_i8_destroy(h_); }
    // copyFrom / copyTo (FR/ascend/AscendIndexInt8Flat.h:90-96; FR/ascend/impl/AscendIndexInt8FlatImpl.cpp:327-431,
    // 580-626): the bytes of IndexScalarQuantizer::codes are the int8 vectors; an IndexIDMap carries the ids
    void copyFrom(const faiss::IndexScalarQuantizer *index) { copyCodes(index, nullptr, 0); }
    void copyFrom(const faiss::IndexIDMap *index)
    {
        if (index == nullptr || index->index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        const auto *sq = dynamic_cast<const faiss::IndexScalarQuantizer *>(index->index);
        if (sq == nullptr) {
            throw FaissException("Invalid sqIndex nullptr.");
        }
        if (!index->id_map.empty() && index->id_map.size() != (size_t)sq->ntotal) {
            throw FaissException("The size of id_map must be equal to ntotal.\n");
        }
        copyCodes(sq, index->id_map.empty() ? nullptr : index->id_map.data(), index->id_map.size());
    }
    void copyTo(faiss::IndexScalarQuantizer *index) const
    {
        if (index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        index->reset();
        index->metric_type = metric_type;
        index->d = d;
        index->code_size = (size_t)d;
        index->is_trained = is_trained;
        if (ntotal > 0) {
            std::vector<int8_t> xb;
            getBase(0, xb);
            index->codes.assign(reinterpret_cast<const uint8_t *>(xb.data()),
                                reinterpret_cast<const uint8_t *>(xb.data()) + xb.size());
        }
        index->ntotal = ntotal;
    }
    void copyTo(faiss::IndexIDMap *index) const
    {
        if (index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        copyTo(dynamic_cast<faiss::IndexScalarQuantizer *>(index->index));
        getIdxMap(0, index->id_map);
        index->d = d;
        index->metric_type = metric_type;
        index->ntotal = ntotal;
    }
    void searchInt32(idx_t n, const int8_t *x, idx_t k, int32_t *distances, idx_t *labels) const
    {
        ixaThrowIfError(flat_i8_search(h_, n, x, k, distances, reinterpret_cast<int64_t *>(labels)));
    }
    // search_with_masks (FR/ascend/AscendIndexInt8Flat.h:98-99), float distances like search()
    void search_with_masks(idx_t n, const int8_t *x, idx_t k, float *distances, idx_t *labels, const void *mask) const
    {
        std::vector<int32_t> tmp((size_t)n * k);
        ixaThrowIfError(flat_i8_search_with_masks(h_, n, x, k, static_cast<const uint8_t *>(mask), tmp.data(),
                                                  reinterpret_cast<int64_t *>(labels)));
        for (size_t i = 0; i < tmp.size(); i++) {
            distances[i] = labels[i] < 0 ? FLT_MAX : (float)tmp[i];
        }
    }
    size_t getBaseSize(int /*deviceId*/ = 0) const { return (size_t)ntotal; }
    void getBase(int /*deviceId*/, std::vector<int8_t> &xb) const
    {
        xb.resize((size_t)ntotal * d);
        if (ntotal > 0) {
            ixaThrowIfError(flat_i8_get_base(h_, 0, ntotal, xb.data()));
        }
    }
    void getIdxMap(int /*deviceId*/, std::vector<idx_t> &idxMap) const
    {
        idxMap.resize((size_t)ntotal);
        if (ntotal > 0) {
            ixaThrowIfError(flat_i8_get_ids(h_, 0, ntotal, reinterpret_cast<int64_t *>(idxMap.data())));
        }
    }
    // remove_ids (FR/ascend/AscendIndexInt8.h:88), as AscendIndexFlat::remove_ids
    size_t remove_ids(const faiss::IDSelector &sel) override
    {
        std::vector<int64_t> ids;
        int64_t imin = 0, imax = 0, removed = 0;
        if (ixaSelectorIds(sel, [this](std::vector<idx_t> &m) { getIdxMap(0, m); }, ids, imin, imax)) {
            ixaThrowIfError(flat_i8_remove_range(h_, imin, imax, &removed));
        } else {
            ixaThrowIfError(flat_i8_remove_ids(h_, (int64_t)ids.size(), ids.data(), &removed));
        }
        int64_t v = 0;
        ixaThrowIfError(flat_i8_ntotal(h_, &v));
        ntotal = v;
        return (size_t)removed;
    }
    void reset()
    {
        ixaThrowIfError(flat_i8_reset(h_));
        ntotal = 0;
    }
    // setPageSize (FR/ascend/AscendIndexInt8Flat.h:101) tunes how many base blocks the reference searches
    // per operator call; the search here streams the whole base through one persistent kernel: accepted, no effect
    void setPageSize(uint16_t /*pageBlockNum*/) {}

protected:
    void copyCodes(const faiss::IndexScalarQuantizer *index, const idx_t *ids, size_t nids)
    {
        if (index == nullptr) {
            throw FaissException("Invalid index nullptr.");
        }
        if (index->d != d || index->metric_type != metric_type) {
            throw FaissException("copyFrom: the source index must have this index's dims and metric");
        }
        (void)nids;
        reset();
        is_trained = index->is_trained;
        if (!index->is_trained || index->codes.empty()) {
            return;
        }
        if (index->codes.size() != (size_t)index->ntotal * (size_t)d) {
            throw FaissException("The size of codes must be equal to ntotal * dim.\n");
        }
        addImpl(index->ntotal, reinterpret_cast<const int8_t *>(index->codes.data()), ids);
    }
    void addImpl(idx_t n, const int8_t *x, const idx_t *ids) override
    {
        ixaThrowIfError(flat_i8_add_with_ids(h_, n, x, reinterpret_cast<const int64_t *>(ids)));
        int64_t v = 0;
        ixaThrowIfError(flat_i8_ntotal(h_, &v));
        ntotal = v;
    }
    void searchImpl(idx_t n, const int8_t *x, idx_t k, float *distances, idx_t *labels) const override
    {
        std::vector<int32_t> tmp((size_t)n * k);
        searchInt32(n, x, k, tmp.data(), labels);
        for (size_t i = 0; i < tmp.size(); i++) {
            distances[i] = labels[i] < 0 ? FLT_MAX : (float)tmp[i];
        }
    }
    flat_i8_index_t *h_ = nullptr;
};

}  // namespace ascend
}  // namespace faiss
