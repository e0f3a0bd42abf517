// Brute-force Flat indexes on one MI355X ("the coarse stage in isolation"):
//   FlatIndex    -- fp32 vectors, L2 or inner product; counterpart of AscendIndexFlat ->
//                   IndexFlatL2Aicpu / IndexFlatIPAicpu (FR/ascendhost/src/index/IndexFlatL2Aicpu.cpp:157-306),
//                   but with fp32 instead of fp16 distances.
//   FlatI8Index  -- int8 vectors, exact int32 L2; counterpart of AscendIndexInt8Flat ->
//                   IndexInt8FlatL2Aicpu (FR/ascendhost/src/index/IndexInt8FlatL2Aicpu.cpp:41-126), without the
//                   reference's final scale-and-round-to-fp16 step.
#pragma once
#include <cstdint>
#include <vector>

#include "common.h"
#include "stream_select.h"

namespace ixa {

constexpr int64_t kMaskPageBytes = (int64_t)256 << 20;   // masks of one query page of a masked search

struct FlatStats {
    double ms_score = 0;        // all score-tile launches of the last search
    double ms_select = 0;       // all selection launches (+ refine / finalisation)
    double ms_total = 0;
    double score_launches = 0;
    double exact_reruns = 0;    // fp32: queries redone from canonical scores of the whole base
};

template <typename T>
class FlatBase {
public:
    FlatBase(int d, int metric, int64_t scratch_bytes);
    virtual ~FlatBase();
    FlatBase(const FlatBase &) = delete;
    FlatBase &operator=(const FlatBase &) = delete;

    int d() const { return d_; }
    int metric() const { return metric_; }
    int64_t ntotal() const { return ntotal_; }
    int64_t scratch_bytes() const { return scratch_bytes_; }
    hipStream_t stream() const { return stream_; }
    void add(int64_t n, const T *x, const int64_t *ids, bool on_device);
    void get_base(int64_t offset, int64_t n, T *out) const;   // host output
    void get_ids(int64_t offset, int64_t n, int64_t *out) const;
    void reset();
    const FlatStats &stats() const { return stats_; }

protected:
    // this index becomes a search view of `owner`: it reads the owner's vectors and ids in place (see IvfpqIndex::borrow_from)
    void borrow_base(const FlatBase &owner)
    {
        ntotal_ = owner.ntotal_;
        capacity_ = owner.capacity_;
        base_.borrow(owner.base_);
        ids_.borrow(owner.ids_);
    }
    void reserve(int64_t n);
    // How the vectors lie in base_: row-major here; FlatI8Index keeps them in matrix-core order (flat_i8.h).
    // new_base <- the first ntotal_ vectors of base_, with room for cap
    virtual void grow_base(int64_t cap);
    // vectors [first, first + n) <- n row-major vectors (host or device memory); queued on stream_
    virtual void store_rows(int64_t first, int64_t n, const T *x, bool on_device);
    // n row-major vectors in host memory <- vectors [offset, offset + n)
    virtual void fetch_rows(int64_t offset, int64_t n, T *out) const;
    // move j: vector moves[2 j + 1] (with id and norm) over vector moves[2 j]; device array of nmoves pairs
    virtual void move_rows(const int64_t *moves, int64_t nmoves, uint32_t *norms);
    // removes the vectors whose id is one of the nv host ids (victims != nullptr) or lies in [imin, imax);
    // norms: the derived class's 4-byte norm per vector, moved along; returns the number removed
    int64_t remove_selected(int64_t nv, const int64_t *victims, int64_t imin, int64_t imax, uint32_t *norms);
    int d_, metric_;
    int64_t scratch_bytes_;
    int64_t ntotal_ = 0, capacity_ = 0;
    hipStream_t stream_ = nullptr;
    hipEvent_t ev_[4] = {nullptr, nullptr, nullptr, nullptr};
    DeviceBuffer<T> base_;
    DeviceBuffer<int64_t> ids_;
    DeviceBuffer<unsigned long long> ws_running_;
    DeviceBuffer<T> ws_x_;
    FlatStats stats_;
};

class FlatIndex : public FlatBase<float> {
public:
    FlatIndex(int d, int metric, int64_t scratch_bytes);
    void add(int64_t n, const float *x, const int64_t *ids, bool on_device);
    void search(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device);
    // host pointers; mask: n rows of ceil(ntotal / 8) bytes, bit set = the vector at that position takes part
    void search_with_masks(int64_t n, const float *x, int64_t k, const uint8_t *mask, float *dist, int64_t *labels);
    int64_t remove_ids(int64_t n, const int64_t *ids);       // host ids; returns the number of vectors removed
    int64_t remove_range(int64_t imin, int64_t imax);        // ids in [imin, imax)
    void reset();
    void borrow_from(const FlatIndex &owner)   // a view serves searches only
    {
        borrow_base(owner);
        norms_.borrow(owner.norms_);
        bmax_ = owner.bmax_;
    }

private:
    // exact results for the listed query rows, from canonical scores of the whole base
    void exact_rows(const float *xd, const std::vector<int64_t> &rows, int64_t k, float *dist_dev, int64_t *labels_dev,
                    const uint8_t *mask_dev, int64_t mask_stride);
    void search_masked(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device,
                       const uint8_t *mask_dev, int64_t mask_stride);
    DeviceBuffer<float> norms_, ws_qn_, ws_dist_;
    StreamSelectWorkspace<float> ws_sel_;
    DeviceBuffer<int32_t> ws_cand_, ws_idx_, ws_flag_;
    DeviceBuffer<int64_t> ws_labels_;
    float bmax_ = 0.f;   // largest base vector norm
};

class FlatI8Index : public FlatBase<int8_t> {
public:
    FlatI8Index(int d, int metric, int64_t scratch_bytes);
    void add(int64_t n, const int8_t *x, const int64_t *ids, bool on_device);
    void search(int64_t n, const int8_t *x, int64_t k, int32_t *dist, int64_t *labels, bool on_device);
    void search_with_masks(int64_t n, const int8_t *x, int64_t k, const uint8_t *mask, int32_t *dist, int64_t *labels);
    int64_t remove_ids(int64_t n, const int64_t *ids);
    int64_t remove_range(int64_t imin, int64_t imax);
    void reset();
    void borrow_from(const FlatI8Index &owner)   // a view serves searches only
    {
        borrow_base(owner);
        norms_.borrow(owner.norms_);
    }

private:
    void search_masked(int64_t n, const int8_t *x, int64_t k, int32_t *dist, int64_t *labels, bool on_device,
                       const uint8_t *mask_dev, int64_t mask_stride);
    void grow_base(int64_t cap) override;
    void store_rows(int64_t first, int64_t n, const int8_t *x, bool on_device) override;
    void fetch_rows(int64_t offset, int64_t n, int8_t *out) const override;
    void move_rows(const int64_t *moves, int64_t nmoves, uint32_t *norms) override;
    void pad_norms();   // INT32_MAX behind the last vector, up to the end of its tile of 256
    // norms_: one per vector, allocated in whole tiles of 256 vectors like the tiled base
    DeviceBuffer<int32_t> norms_, ws_qn_, ws_dist_;
    mutable DeviceBuffer<int8_t> ws_rows_;   // row-major staging of vectors on their way in or out
    StreamSelectWorkspace<int32_t> ws_sel_;
    DeviceBuffer<int64_t> ws_labels_;
};

// dst[0:bytes] = src[0:bytes] on the device with a plain copy kernel (traffic-counter yardstick).
void launch_copy_probe(const void *src, void *dst, int64_t bytes);
// Average duration (ms) of one plain streaming read of src[0:bytes] over `passes` passes.
double launch_read_probe(const void *src, int64_t bytes, int passes);

}  // namespace ixa
