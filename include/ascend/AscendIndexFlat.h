// Header-only C++ faces of the Flat paths with the reference's class shapes:
//   faiss::ascend::AscendIndexFlat / AscendIndexFlatL2   (FR/ascend/AscendIndexFlat.h:48-90)
//   faiss::ascend::AscendIndexInt8Flat                   (FR/ascend/AscendIndexInt8.h:53-96, AscendIndexInt8Flat.h)
// forwarding to the C ABI (include/indexsdk_amd.h).
#pragma once
#include <cfloat>
#include <vector>

#include "AscendIndexIVFPQ.h"

namespace faiss {
namespace ascend {

class AscendIndexFlat : public faiss::Index {
public:
    AscendIndexFlat(int dims, faiss::MetricType metric, int64_t resourceSize = 0) : faiss::Index(dims, metric)
    {
        ixaThrowIfError(flat_create(dims, (int)metric, resourceSize, &h_));
    }
    virtual ~AscendIndexFlat() { flat_destroy(h_); }
    AscendIndexFlat(const AscendIndexFlat &) = delete;
    AscendIndexFlat &operator=(const AscendIndexFlat &) = delete;
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
    void reset() override
    {
        ixaThrowIfError(flat_reset(h_));
        ntotal = 0;
    }
    size_t getBaseSize(int /*deviceId*/ = 0) const { return (size_t)ntotal; }
    void getBase(int /*deviceId*/, std::vector<float> &xb) const
    {
        xb.resize((size_t)ntotal * d);
        ixaThrowIfError(flat_get_base(h_, 0, ntotal, xb.data()));
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
    explicit AscendIndexFlatL2(int dims, int64_t resourceSize = 0) : AscendIndexFlat(dims, faiss::METRIC_L2, resourceSize)
    {
    }
};

// int8 vectors; L2 only.  search() keeps the reference's float signature (exact below 2^24,
// rounded to nearest above); searchInt32() returns the exact int32 distances.
class AscendIndexInt8Flat {
public:
    using idx_t = faiss::idx_t;
    AscendIndexInt8Flat(int dims, faiss::MetricType metric = faiss::METRIC_L2, int64_t resourceSize = 0) : d(dims)
    {
        ixaThrowIfError(flat_i8_create(dims, (int)metric, resourceSize, &h_));
    }
    virtual ~AscendIndexInt8Flat() { flat_i8_destroy(h_); }
    AscendIndexInt8Flat(const AscendIndexInt8Flat &) = delete;
    AscendIndexInt8Flat &operator=(const AscendIndexInt8Flat &) = delete;
    void add(idx_t n, const int8_t *x) { add_with_ids(n, x, nullptr); }
    void add_with_ids(idx_t n, const int8_t *x, const idx_t *ids)
    {
        ixaThrowIfError(flat_i8_add_with_ids(h_, n, x, reinterpret_cast<const int64_t *>(ids)));
        int64_t v = 0;
        ixaThrowIfError(flat_i8_ntotal(h_, &v));
        ntotal = v;
    }
    void searchInt32(idx_t n, const int8_t *x, idx_t k, int32_t *distances, idx_t *labels) const
    {
        ixaThrowIfError(flat_i8_search(h_, n, x, k, distances, reinterpret_cast<int64_t *>(labels)));
    }
    void search(idx_t n, const int8_t *x, idx_t k, float *distances, idx_t *labels) const
    {
        std::vector<int32_t> tmp((size_t)n * k);
        searchInt32(n, x, k, tmp.data(), labels);
        for (size_t i = 0; i < tmp.size(); i++) {
            distances[i] = labels[i] < 0 ? FLT_MAX : (float)tmp[i];
        }
    }
    void reset()
    {
        ixaThrowIfError(flat_i8_reset(h_));
        ntotal = 0;
    }
    int d;
    idx_t ntotal = 0;

protected:
    flat_i8_index_t *h_ = nullptr;
};

}  // namespace ascend
}  // namespace faiss
