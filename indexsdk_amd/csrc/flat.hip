// Brute-force Flat search: fp32 (scores on the fp32 matrix cores, exact refine) and int8 (exact
// int32 L2 on the int8 matrix cores).  See flat_index.h for the reference counterparts.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <unordered_map>
#include <vector>

#include "coarse.h"
#include "flat_i8.h"
#include "flat_index.h"
#include "stream_select.h"
#include "topk.h"

namespace ixa {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int64_t kMaxN = 1000000000;
constexpr int64_t kMaxK = 2048;

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

// |row|^2 of int8 rows in int32 (FR/ascenddaemon/impl/IndexInt8Flat.cpp:938-967).  One wavefront
// per row; integer sums are order-free.
__global__ __launch_bounds__(256) void sqnorm_rows_i8_kernel(const int8_t *__restrict__ x, int64_t n, int d,
                                                             int32_t *__restrict__ out)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) {
        return;
    }
    const int8_t *p = x + row * d;
    int32_t s = 0;
    for (int j = lane; j < d; j += 64) {
        const int32_t v = p[j];
        s += v * v;
    }
    for (int o = 32; o > 0; o >>= 1) {
        s += __shfl_down(s, o);
    }
    if (lane == 0) {
        out[row] = s;
    }
}

}  // namespace

namespace {

// keys -> (distance, label); label = ids[position].
template <typename S, typename OutT>
__global__ __launch_bounds__(256) void finish_keys_kernel(const key_t *__restrict__ keys, int64_t n, int metric,
                                                          const int64_t *__restrict__ ids, OutT pad,
                                                          OutT *__restrict__ out_dist, int64_t *__restrict__ out_labels)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) {
        return;
    }
    const key_t kk = keys[i];
    if (kk == kEmptyKey) {
        out_dist[i] = pad;
        out_labels[i] = -1;
        return;
    }
    const S v = key_score_as<S>(kk);
    out_dist[i] = metric == kMetricL2 ? (OutT)v : (OutT)(-v);
    out_labels[i] = ids[key_index(kk)];
}

// largest value of a non-negative float array: the bit patterns order like the values
__global__ __launch_bounds__(256) void max_bits_kernel(const float *__restrict__ v, int64_t n, uint32_t *__restrict__ out)
{
    uint32_t m = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const uint32_t b = __float_as_uint(v[i]);
        m = b > m ? b : m;
    }
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t t = __shfl_down(m, o);
        m = t > m ? t : m;
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMax(out, m);
    }
}

__global__ __launch_bounds__(256) void gather_rows_f32_kernel(const float *__restrict__ x, const int64_t *__restrict__ idx,
                                                              int64_t n, int d, float *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n * d) {
        out[e] = x[idx[e / d] * d + e % d];
    }
}

// result rows idx[i] <- rows i of the compact results
__global__ __launch_bounds__(256) void scatter_result_rows_kernel(const float *__restrict__ dist,
                                                                  const int64_t *__restrict__ labels,
                                                                  const int64_t *__restrict__ idx, int64_t n, int k,
                                                                  float *__restrict__ out_dist,
                                                                  int64_t *__restrict__ out_labels)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n * k) {
        const int64_t o = idx[e / k] * k + e % k;
        out_dist[o] = dist[e];
        out_labels[o] = labels[e];
    }
}

__global__ __launch_bounds__(256) void map_labels_kernel(const int32_t *__restrict__ idx, int64_t n,
                                                         const int64_t *__restrict__ ids, int64_t *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        out[i] = idx[i] < 0 ? -1 : ids[idx[i]];
    }
}

// Positions of the vectors a removal selects: those whose id is among the sorted `victims` (binary search),
// or, without a victim list, inside [imin, imax).  Every hit takes a slot of `out` from an atomic counter
// (positions arrive in no particular order); with out == nullptr the launch only counts.
__global__ __launch_bounds__(256) void select_positions_kernel(const int64_t *__restrict__ ids, int64_t n,
                                                               const int64_t *__restrict__ victims, int64_t nv,
                                                               int64_t imin, int64_t imax, int64_t *__restrict__ out,
                                                               int64_t cap, unsigned long long *__restrict__ count)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int64_t id = ids[i];
    bool hit;
    if (victims == nullptr) {
        hit = id >= imin && id < imax;
    } else {
        int64_t lo = 0, hi = nv;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (victims[mid] < id) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        hit = lo < nv && victims[lo] == id;
    }
    if (hit) {
        const unsigned long long slot = atomicAdd(count, 1ull);
        if (out != nullptr && (int64_t)slot < cap) {
            out[slot] = i;
        }
    }
}

// Move j copies row moves[2 j + 1] (vector, id, norm) over row moves[2 j].  Sources lie past the new end of
// the base and destinations before it, so no move reads what another writes.
template <typename T>
__global__ __launch_bounds__(128) void move_rows_kernel(T *__restrict__ base, int64_t *__restrict__ ids,
                                                        uint32_t *__restrict__ norms,
                                                        const int64_t *__restrict__ moves, int d)
{
    const int64_t dst = moves[2 * (int64_t)blockIdx.x], src = moves[2 * (int64_t)blockIdx.x + 1];
    for (int t = threadIdx.x; t < d; t += 128) {
        base[dst * d + t] = base[src * d + t];
    }
    if (threadIdx.x == 0) {
        ids[dst] = ids[src];
        if (norms != nullptr) {
            norms[dst] = norms[src];
        }
    }
}

__global__ __launch_bounds__(256) void iota_ids_kernel(int64_t *out, int64_t n, int64_t base)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        out[i] = base + i;
    }
}

}  // namespace

// Plain 16-byte-per-lane copy of known size: the yardstick that HBM traffic counters of the other
// kernels are scaled by.
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                                                         int64_t n16)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) {
        dst[i] = src[i];
    }
}

// Plain streaming read: the lanes only fold what they load, and the impossible comparison keeps the loads
// alive without a store.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4 *__restrict__ src, int64_t n16,
                                                         uint32_t *__restrict__ sink)
{
    uint32_t acc = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) {
        const uint4 v = src[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9e3779b9u && sink) {
        *sink = acc;
    }
}

double launch_read_probe(const void *src, int64_t bytes, int passes)
{
    IXA_REQUIRE(src && bytes > 0 && bytes % 16 == 0 && passes >= 1 && passes <= 1000, kErrInvalidParam,
                "read probe needs a multiple of 16 bytes and 1..1000 passes");
    hipEvent_t e0 = nullptr, e1 = nullptr;
    IXA_HIP(hipEventCreate(&e0));
    IXA_HIP(hipEventCreate(&e1));
    float ms = 0.f;
    // eight workgroups per CU: measured best of 4 / 8 / 16 / 32 on an 8 GiB buffer
    hipLaunchKernelGGL(read_probe_kernel, dim3(256 * 8), dim3(256), 0, nullptr, static_cast<const uint4 *>(src),
                       bytes / 16, static_cast<uint32_t *>(nullptr));   // warm-up
    hipError_t err = hipEventRecord(e0, nullptr);
    for (int p = 0; p < passes && err == hipSuccess; p++) {
        hipLaunchKernelGGL(read_probe_kernel, dim3(256 * 8), dim3(256), 0, nullptr, static_cast<const uint4 *>(src),
                           bytes / 16, static_cast<uint32_t *>(nullptr));
    }
    if (err == hipSuccess) {
        err = hipEventRecord(e1, nullptr);
    }
    if (err == hipSuccess) {
        err = hipEventSynchronize(e1);
    }
    if (err == hipSuccess) {
        err = hipEventElapsedTime(&ms, e0, e1);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    IXA_HIP(err);
    IXA_HIP(hipGetLastError());
    return (double)ms / passes;
}

void launch_copy_probe(const void *src, void *dst, int64_t bytes)
{
    IXA_REQUIRE(src && dst && bytes > 0 && bytes % 16 == 0, kErrInvalidParam, "copy probe needs a multiple of 16 bytes");
    hipLaunchKernelGGL(copy_probe_kernel, dim3(256 * 16), dim3(256), 0, nullptr, static_cast<const uint4 *>(src),
                       static_cast<uint4 *>(dst), bytes / 16);
    IXA_HIP(hipGetLastError());
    IXA_HIP(hipDeviceSynchronize());
}

// -------------------------------------------------------------------------------------------------

template <typename T>
FlatBase<T>::FlatBase(int d, int metric, int64_t scratch_bytes) : d_(d), metric_(metric), scratch_bytes_(scratch_bytes)
{
    IXA_REQUIRE(metric == kMetricL2 || metric == kMetricInnerProduct, kErrInvalidParam, "Unsupported metric type");
    IXA_REQUIRE(d >= 1 && d <= 4096, kErrInvalidParam, "Unsupported dims: %d\n", d);
    IXA_REQUIRE(scratch_bytes >= (1 << 20), kErrInvalidParam, "scratch_bytes must be at least 1 MiB");
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    IXA_REQUIRE(e == hipSuccess && ndev > 0, kErrIndexNotInit,
                "no HIP device available (%s): this library has no CPU path", hipGetErrorString(e));
    IXA_HIP(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    for (auto &ev : ev_) {
        IXA_HIP(hipEventCreate(&ev));
    }
}

template <typename T>
FlatBase<T>::~FlatBase()
{
    if (stream_) {
        (void)hipStreamSynchronize(stream_);
    }
    for (auto &ev : ev_) {
        if (ev) {
            (void)hipEventDestroy(ev);
        }
    }
    if (stream_) {
        (void)hipStreamDestroy(stream_);
    }
}

// Grows the base / id arrays geometrically, keeping their content.
template <typename T>
void FlatBase<T>::reserve(int64_t n)
{
    if (n <= capacity_) {
        return;
    }
    const int64_t cap = std::max<int64_t>(n, capacity_ + capacity_ / 2);
    DeviceBuffer<int64_t> ni((size_t)cap);
    if (ntotal_ > 0) {
        IXA_HIP(hipMemcpyAsync(ni.data(), ids_.data(), (size_t)ntotal_ * 8, hipMemcpyDeviceToDevice, stream_));
    }
    grow_base(cap);   // waits for the stream before it releases the old base
    ids_ = std::move(ni);
    capacity_ = cap;
}

template <typename T>
void FlatBase<T>::grow_base(int64_t cap)
{
    DeviceBuffer<T> nb((size_t)cap * d_);
    if (ntotal_ > 0) {
        IXA_HIP(hipMemcpyAsync(nb.data(), base_.data(), (size_t)ntotal_ * d_ * sizeof(T), hipMemcpyDeviceToDevice,
                               stream_));
    }
    sync_stream(stream_);
    base_ = std::move(nb);
}

template <typename T>
void FlatBase<T>::store_rows(int64_t first, int64_t n, const T *x, bool on_device)
{
    IXA_HIP(hipMemcpyAsync(base_.data() + first * d_, x, (size_t)n * d_ * sizeof(T),
                           on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice, stream_));
}

template <typename T>
void FlatBase<T>::fetch_rows(int64_t offset, int64_t n, T *out) const
{
    IXA_HIP(hipMemcpyAsync(out, base_.data() + offset * d_, (size_t)n * d_ * sizeof(T), hipMemcpyDeviceToHost, stream_));
    sync_stream(stream_);
}

// add / add_with_ids (FR/ascend/AscendIndex.h:66-71); ids default to ntotal + i.
template <typename T>
void FlatBase<T>::add(int64_t n, const T *x, const int64_t *ids, bool on_device)
{
    IXA_REQUIRE(x, kErrInvalidParam, "x can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(ntotal_ + n < ((int64_t)1 << 32) - 1, kErrInvalidParam, "index would exceed the 32-bit row space");
    reserve(ntotal_ + n);
    const hipMemcpyKind kind = on_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
    store_rows(ntotal_, n, x, on_device);
    if (ids) {
        IXA_HIP(hipMemcpyAsync(ids_.data() + ntotal_, ids, (size_t)n * 8, kind, stream_));
    } else {
        hipLaunchKernelGGL(iota_ids_kernel, dim3(blocks_for(n)), dim3(256), 0, stream_, ids_.data() + ntotal_, n,
                           ntotal_);
    }
    sync_stream(stream_);
    ntotal_ += n;
}

template <typename T>
void FlatBase<T>::get_base(int64_t offset, int64_t n, T *out) const
{
    IXA_REQUIRE(offset >= 0 && n >= 0 && offset + n <= ntotal_ && (n == 0 || out), kErrInvalidParam,
                "range [%ld, %ld) is outside the index (ntotal %ld)", (long)offset, (long)(offset + n), (long)ntotal_);
    if (n) {
        fetch_rows(offset, n, out);
    }
}

template <typename T>
void FlatBase<T>::get_ids(int64_t offset, int64_t n, int64_t *out) const
{
    IXA_REQUIRE(offset >= 0 && n >= 0 && offset + n <= ntotal_ && (n == 0 || out), kErrInvalidParam,
                "range [%ld, %ld) is outside the index (ntotal %ld)", (long)offset, (long)(offset + n), (long)ntotal_);
    if (n) {
        IXA_HIP(hipMemcpyAsync(out, ids_.data() + offset, (size_t)n * 8, hipMemcpyDeviceToHost, stream_));
        sync_stream(stream_);
    }
}

// remove_ids (FR/ascend/impl/AscendIndexImpl.cpp:208-270 picks the positions whose id the selector names,
// FR/ascenddaemon/impl/Index.cpp:86-113 removes them): the positions are visited from the highest to the
// lowest and each is overwritten with the vector that is last at that moment, which then leaves the end.
// The device does the outcome of that sequence in one launch: every removed position below the new end
// receives the vector the sequence leaves there (always one from at or past the new end), everything else
// stays where it is.  victims == nullptr selects by range.
template <typename T>
int64_t FlatBase<T>::remove_selected(int64_t nv, const int64_t *victims, int64_t imin, int64_t imax, uint32_t *norms)
{
    IXA_REQUIRE(nv >= 0 && nv < kMaxN && (nv == 0 || victims), kErrInvalidParam, "ids can not be nullptr.");
    if (ntotal_ == 0 || (victims == nullptr ? imin >= imax : nv == 0)) {
        return 0;
    }
    DeviceBuffer<int64_t> victims_dev;
    std::vector<int64_t> sorted;   // source of an asynchronous copy: lives until the stream has been waited for
    if (victims) {
        sorted.assign(victims, victims + nv);
        std::sort(sorted.begin(), sorted.end());
        sorted.erase(std::unique(sorted.begin(), sorted.end()), sorted.end());
        nv = (int64_t)sorted.size();
        victims_dev.upload(sorted.data(), sorted.size(), stream_);
    }
    DeviceBuffer<unsigned long long> count(1);
    unsigned long long hits = 0;
    IXA_HIP(hipMemsetAsync(count.data(), 0, 8, stream_));
    hipLaunchKernelGGL(select_positions_kernel, dim3(blocks_for(ntotal_)), dim3(256), 0, stream_, ids_.data(), ntotal_,
                       victims ? victims_dev.data() : nullptr, nv, imin, imax, (int64_t *)nullptr, (int64_t)0,
                       count.data());
    count.download(&hits, 1, stream_);
    if (hits == 0) {
        return 0;
    }
    if ((int64_t)hits == ntotal_) {   // everything leaves: nothing to move
        ntotal_ = 0;
        return (int64_t)hits;
    }
    DeviceBuffer<int64_t> pos_dev((size_t)hits);
    IXA_HIP(hipMemsetAsync(count.data(), 0, 8, stream_));
    hipLaunchKernelGGL(select_positions_kernel, dim3(blocks_for(ntotal_)), dim3(256), 0, stream_, ids_.data(), ntotal_,
                       victims ? victims_dev.data() : nullptr, nv, imin, imax, pos_dev.data(), (int64_t)hits,
                       count.data());
    std::vector<int64_t> gone((size_t)hits);
    pos_dev.download(gone.data(), gone.size(), stream_);
    std::sort(gone.begin(), gone.end());
    const int64_t left = ntotal_ - (int64_t)hits;
    // The sequence is replayed on the host with only the overwritten positions recorded (a vector can move
    // several times: into a hole of the tail first, on into a lower hole later); what finally matters is
    // which original vector each hole below the new end holds.  Those vectors all come from positions at
    // or past the new end, each exactly once.
    std::unordered_map<int64_t, int64_t> holds;   // position -> original position of the vector now there
    holds.reserve(gone.size());
    auto at = [&](int64_t p) {
        const auto it = holds.find(p);
        return it == holds.end() ? p : it->second;
    };
    int64_t cur = ntotal_;
    for (int64_t g = (int64_t)gone.size() - 1; g >= 0; g--, cur--) {
        const int64_t hole = gone[(size_t)g];
        if (hole != cur - 1) {
            holds[hole] = at(cur - 1);
        }
    }
    std::vector<int64_t> moves;
    for (size_t g = 0; g < gone.size() && gone[g] < left; g++) {
        const int64_t src = holds.at(gone[g]);
        IXA_REQUIRE(src >= left && src < ntotal_, kErrInner, "remove: hole %ld would be filled from position %ld",
                    (long)gone[g], (long)src);
        moves.push_back(gone[g]);
        moves.push_back(src);
    }
    if (!moves.empty()) {
        DeviceBuffer<int64_t> moves_dev;
        moves_dev.upload(moves.data(), moves.size(), stream_);
        move_rows(moves_dev.data(), (int64_t)(moves.size() / 2), norms);
        sync_stream(stream_);   // moves_dev is freed on return
    }
    ntotal_ = left;
    return (int64_t)hits;
}

template <typename T>
void FlatBase<T>::move_rows(const int64_t *moves, int64_t nmoves, uint32_t *norms)
{
    hipLaunchKernelGGL((move_rows_kernel<T>), dim3((unsigned)nmoves), dim3(128), 0, stream_, base_.data(), ids_.data(),
                       norms, moves, d_);
}

template <typename T>
void FlatBase<T>::reset()
{
    sync_stream(stream_);
    base_.release();
    ids_.release();
    ntotal_ = capacity_ = 0;
}

template class FlatBase<float>;
template class FlatBase<int8_t>;

// ---- fp32 ---------------------------------------------------------------------------------------

FlatIndex::FlatIndex(int d, int metric, int64_t scratch_bytes) : FlatBase<float>(d, metric, scratch_bytes) {}

void FlatIndex::add(int64_t n, const float *x, const int64_t *ids, bool on_device)
{
    const int64_t before = ntotal_;
    FlatBase<float>::add(n, x, ids, on_device);
    // norms of the whole base are kept in one array; recompute the tail (left-to-right fp32)
    DeviceBuffer<float> nn((size_t)capacity_);
    if (before > 0) {
        IXA_HIP(hipMemcpyAsync(nn.data(), norms_.data(), (size_t)before * 4, hipMemcpyDeviceToDevice, stream_));
    }
    launch_sqnorm_rows(base_.data() + before * d_, n, d_, nn.data() + before, stream_);
    // largest norm of the base (the error bound of the approximate scores is proportional to it)
    DeviceBuffer<uint32_t> mx(1);
    IXA_HIP(hipMemsetAsync(mx.data(), 0, 4, stream_));
    hipLaunchKernelGGL(max_bits_kernel, dim3((unsigned)std::min<int64_t>(1024, (n + 255) / 256)), dim3(256), 0, stream_,
                       nn.data() + before, n, mx.data());
    uint32_t bits = 0;
    mx.download(&bits, 1, stream_);
    float sq;
    std::memcpy(&sq, &bits, 4);
    bmax_ = std::max(bmax_, std::sqrt(sq));
    norms_ = std::move(nn);
}

// Exact plan of last resort (queries whose candidate list cannot be proven complete): canonical scores
// of the whole base, chunk by chunk, with an exact running selection.
void FlatIndex::exact_rows(const float *xd, const std::vector<int64_t> &rows, int64_t k, float *dist_dev,
                           int64_t *labels_dev, const uint8_t *mask_dev, int64_t mask_stride)
{
    const int64_t total_rows = (int64_t)rows.size();
    DeviceBuffer<int64_t> rows_dev;
    rows_dev.upload(rows.data(), rows.size(), stream_);
    DeviceBuffer<float> xsub, qn, scores, dsub;
    DeviceBuffer<unsigned long long> running;
    DeviceBuffer<int64_t> lsub;
    for (int64_t r0 = 0; r0 < total_rows; r0 += 4096) {
        const int64_t m = std::min<int64_t>(4096, total_rows - r0);
        const int64_t cols = std::max<int64_t>(4096, std::min<int64_t>(ntotal_, scratch_bytes_ / (4 * m)));
        xsub.resize((size_t)m * d_);
        qn.resize((size_t)m);
        scores.resize((size_t)m * cols);
        running.resize((size_t)m * k);
        dsub.resize((size_t)m * k);
        lsub.resize((size_t)m * k);
        hipLaunchKernelGGL(gather_rows_f32_kernel, dim3(blocks_for(m * d_)), dim3(256), 0, stream_, xd, rows_dev.data() + r0,
                           m, d_, xsub.data());
        launch_sqnorm_rows(xsub.data(), m, d_, qn.data(), stream_);
        IXA_HIP(hipMemsetAsync(running.data(), 0xff, running.bytes(), stream_));
        for (int64_t c0 = 0; c0 < ntotal_; c0 += cols) {
            const int64_t nc = std::min(cols, ntotal_ - c0);
            launch_canonical_scores(xsub.data(), m, base_.data() + c0 * d_, nc, d_, qn.data(), norms_.data() + c0, metric_,
                                    scores.data(), nc, stream_);
            if (mask_dev) {
                launch_apply_mask(scores.data(), m, nc, nc, mask_dev, mask_stride, rows_dev.data() + r0, c0, stream_);
            }
            launch_select_rows(scores.data(), m, nc, nc, (int)k, nullptr, c0, running.data(), stream_);
        }
        if (mask_dev) {
            launch_drop_worst_keys_f32(running.data(), m * k, stream_);
        }
        const float pad = metric_ == kMetricL2 ? 3.402823466e+38f : -3.402823466e+38f;
        hipLaunchKernelGGL((finish_keys_kernel<float, float>), dim3(blocks_for(m * k)), dim3(256), 0, stream_,
                           running.data(), m * k, metric_, ids_.data(), pad, dsub.data(), lsub.data());
        hipLaunchKernelGGL(scatter_result_rows_kernel, dim3(blocks_for(m * k)), dim3(256), 0, stream_, dsub.data(),
                           lsub.data(), rows_dev.data() + r0, m, (int)k, dist_dev, labels_dev);
    }
    sync_stream(stream_);   // the temporaries above are freed on return
}

void FlatIndex::reset()
{
    FlatBase<float>::reset();
    norms_.release();
}

int64_t FlatIndex::remove_ids(int64_t n, const int64_t *ids)
{
    IXA_REQUIRE(n >= 0 && (n == 0 || ids), kErrInvalidParam, "ids can not be nullptr.");
    return remove_selected(n, ids, 0, 0, reinterpret_cast<uint32_t *>(norms_.data()));
}

int64_t FlatIndex::remove_range(int64_t imin, int64_t imax)
{
    return remove_selected(0, nullptr, imin, imax, reinterpret_cast<uint32_t *>(norms_.data()));
}

// search (FR/ascendhost/src/index/IndexFlatL2Aicpu.cpp:157-306): the base is walked in row chunks;
// every chunk's scores are selected into a running top-(k + slack) per query, and the survivors
// are re-evaluated in the canonical scalar arithmetic before the final top-k is written.
void FlatIndex::search(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device)
{
    search_masked(n, x, k, dist, labels, on_device, nullptr, 0);
}

// search_with_masks (FR/ascend/AscendIndexFlat.h:78-82; FR/ascend/impl/AscendIndexFlatImpl.cpp:461-511): row i of
// the mask (ceil(ntotal / 8) bytes, host memory) says which base vectors query i may return: bit p % 8 of
// byte p / 8 set = the vector at position p takes part.  Queries go in pages whose masks fit a bounded
// device buffer.
void FlatIndex::search_with_masks(int64_t n, const float *x, int64_t k, const uint8_t *mask, float *dist, int64_t *labels)
{
    IXA_REQUIRE(mask, kErrInvalidParam, "mask cannot be nullptr.");
    IXA_REQUIRE(x && dist && labels, kErrInvalidParam, "x, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    const int64_t stride = (ntotal_ + 7) / 8;
    if (stride == 0) {
        search_masked(n, x, k, dist, labels, false, nullptr, 0);
        return;
    }
    const int64_t page = std::max<int64_t>(1, std::min<int64_t>(n, kMaskPageBytes / stride));
    DeviceBuffer<uint8_t> mask_dev;
    for (int64_t q0 = 0; q0 < n; q0 += page) {
        const int64_t nq = std::min(page, n - q0);
        mask_dev.upload(mask + q0 * stride, (size_t)(nq * stride), stream_);
        search_masked(nq, x + q0 * d_, k, dist + q0 * k, labels + q0 * k, false, mask_dev.data(), stride);
    }
}

void FlatIndex::search_masked(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device,
                              const uint8_t *mask_dev, int64_t mask_stride)
{
    IXA_REQUIRE(x && dist && labels, kErrInvalidParam, "x, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(k > 0 && k <= kMaxK, kErrInvalidParam, "k must be > 0 and <= %ld", (long)kMaxK);
    const float *xd = x;
    if (!on_device) {
        ws_x_.upload(x, (size_t)n * d_, stream_);
        xd = ws_x_.data();
    }
    float *dd = dist;
    int64_t *ld = labels;
    if (!on_device) {
        ws_dist_.resize((size_t)n * k);
        ws_labels_.resize((size_t)n * k);
        dd = ws_dist_.data();
        ld = ws_labels_.data();
    }
    const int ncand = (int)std::min<int64_t>(std::max<int64_t>(ntotal_, 1), k + 8 + k / 8);
    ws_qn_.resize((size_t)n);
    ws_running_.resize((size_t)n * ncand);
    ws_cand_.resize((size_t)n * ncand);
    ws_idx_.resize((size_t)n * k);
    IXA_HIP(hipEventRecord(ev_[0], stream_));
    launch_sqnorm_rows(xd, n, d_, ws_qn_.data(), stream_);
    const int launches = stream_select_f32(xd, n, base_.data(), ntotal_, d_, ws_qn_.data(), norms_.data(), metric_,
                                           ncand, ws_running_.data(), ws_sel_, scratch_bytes_, stream_, mask_dev,
                                           mask_stride);
    if (mask_dev) {
        launch_drop_worst_keys_f32(ws_running_.data(), n * ncand, stream_);   // vectors the query leaves out
    }
    IXA_HIP(hipEventRecord(ev_[1], stream_));
    launch_keys_to_idx(ws_running_.data(), n * ncand, ws_cand_.data(), stream_);
    launch_refine(xd, n, base_.data(), d_, ws_qn_.data(), norms_.data(), metric_, ws_cand_.data(), ncand,
                  (int)std::min<int64_t>(k, ncand), (int)k, ws_idx_.data(), dd, stream_);
    hipLaunchKernelGGL(map_labels_kernel, dim3(blocks_for(n * k)), dim3(256), 0, stream_, ws_idx_.data(), n * k,
                       ids_.data(), ld);
    // Proof that no base vector outside a query's candidate list can reach its k-th exact score; the
    // approximate scores are fp32 matrix-core sums: they and the canonical left-to-right sums are each
    // within (d + 1) 2^-24 sum |x_i y_i| of the exact dot product (a few units added for second-order
    // terms); an L2 score holds two dot products and three further roundings of numbers no larger
    // than (|q| + |b|)^2.  Queries without proof are redone exactly.
    stats_.exact_reruns = 0;
    if (ncand < ntotal_) {
        const float u = 5.9604645e-8f;
        const float err_scale = (metric_ == kMetricL2 ? 2.0f : 1.0f) * (float)(2 * d_ + 8) * u;
        const float round_scale = metric_ == kMetricL2 ? 4.0f * u : 0.0f;
        ws_flag_.resize((size_t)n + 1);
        IXA_HIP(hipMemsetAsync(ws_flag_.data(), 0, sizeof(int32_t), stream_));
        launch_verify_superset(ws_running_.data(), ncand, dd, (int)k, ws_qn_.data(), bmax_, err_scale, round_scale, metric_,
                               n, ws_flag_.data(), stream_);
        int32_t nfail = 0;
        ws_flag_.download(&nfail, 1, stream_);
        if (nfail > 0) {
            std::vector<int32_t> rows32((size_t)nfail);
            IXA_HIP(hipMemcpyAsync(rows32.data(), ws_flag_.data() + 1, (size_t)nfail * 4, hipMemcpyDeviceToHost, stream_));
            sync_stream(stream_);
            std::sort(rows32.begin(), rows32.end());
            exact_rows(xd, std::vector<int64_t>(rows32.begin(), rows32.end()), k, dd, ld, mask_dev, mask_stride);
            stats_.exact_reruns = nfail;
        }
    }
    IXA_HIP(hipEventRecord(ev_[2], stream_));
    sync_stream(stream_);
    if (!on_device) {
        ws_dist_.download(dist, (size_t)n * k, stream_);
        ws_labels_.download(labels, (size_t)n * k, stream_);
    }
    float a = 0, b = 0;
    IXA_HIP(hipEventElapsedTime(&a, ev_[0], ev_[1]));
    IXA_HIP(hipEventElapsedTime(&b, ev_[1], ev_[2]));
    stats_.ms_score = a;
    stats_.ms_select = b;
    stats_.ms_total = a + b;
    stats_.score_launches = launches;
}

// ---- int8 ---------------------------------------------------------------------------------------

FlatI8Index::FlatI8Index(int d, int metric, int64_t scratch_bytes) : FlatBase<int8_t>(d, metric, scratch_bytes)
{
    // the reference's Int8Flat serves L2 and cosine; only the exact-int32 L2 path is built here
    IXA_REQUIRE(metric == kMetricL2, kErrInvalidParam, "Unsupported metric type");
}

// The base lives in matrix-core order (flat_i8.h); vectors come in and go out row-major through ws_rows_.
void FlatI8Index::grow_base(int64_t cap)
{
    DeviceBuffer<int8_t> nb(i8_tiled_bytes(cap, d_));
    DeviceBuffer<int32_t> nn((size_t)round_up(cap, kI8TileRows));
    if (ntotal_ > 0) {
        // blocks of 32 vectors are contiguous: the blocks that hold the first ntotal_ vectors
        IXA_HIP(hipMemcpyAsync(nb.data(), base_.data(), (size_t)round_up(ntotal_, kI8BlockRows) * i8_padded_dim(d_),
                               hipMemcpyDeviceToDevice, stream_));
        IXA_HIP(hipMemcpyAsync(nn.data(), norms_.data(), (size_t)ntotal_ * 4, hipMemcpyDeviceToDevice, stream_));
    }
    sync_stream(stream_);
    base_ = std::move(nb);
    norms_ = std::move(nn);
}

void FlatI8Index::store_rows(int64_t first, int64_t n, const int8_t *x, bool on_device)
{
    // host vectors pass through a bounded staging buffer, piece by piece
    const int64_t piece = on_device ? n : std::max<int64_t>(1, ((int64_t)256 << 20) / d_);
    for (int64_t o = 0; o < n; o += piece) {
        const int64_t m = std::min(piece, n - o);
        const int8_t *xd = x + o * d_;
        if (!on_device) {
            if (o > 0) {
                sync_stream(stream_);   // the kernels that read the previous piece
            }
            ws_rows_.upload(xd, (size_t)m * d_, stream_);
            xd = ws_rows_.data();
        }
        launch_i8_tile_rows(xd, m, d_, base_.data(), first + o, stream_);
        hipLaunchKernelGGL(sqnorm_rows_i8_kernel, dim3((unsigned)((m + 3) / 4)), dim3(256), 0, stream_, xd, m, d_,
                           norms_.data() + first + o);
    }
}

void FlatI8Index::fetch_rows(int64_t offset, int64_t n, int8_t *out) const
{
    // in pieces, so that the staging buffer stays small whatever the caller asks for
    const int64_t piece = std::max<int64_t>(1, ((int64_t)64 << 20) / d_);
    for (int64_t o = 0; o < n; o += piece) {
        const int64_t m = std::min(piece, n - o);
        ws_rows_.resize((size_t)m * d_);
        launch_i8_untile_rows(base_.data(), offset + o, m, d_, ws_rows_.data(), stream_);
        ws_rows_.download(out + o * d_, (size_t)m * d_, stream_);
    }
}

void FlatI8Index::move_rows(const int64_t *moves, int64_t nmoves, uint32_t *norms)
{
    launch_i8_move_rows(base_.data(), d_, ids_.data(), reinterpret_cast<int32_t *>(norms), moves, nmoves, stream_);
}

void FlatI8Index::pad_norms()
{
    if (capacity_ > 0) {
        launch_i8_pad_norms(norms_.data(), ntotal_, round_up(std::max<int64_t>(ntotal_, 1), kI8TileRows), stream_);
    }
}

void FlatI8Index::add(int64_t n, const int8_t *x, const int64_t *ids, bool on_device)
{
    FlatBase<int8_t>::add(n, x, ids, on_device);   // store_rows computes the norms of what it stores
    pad_norms();
    sync_stream(stream_);
}

int64_t FlatI8Index::remove_ids(int64_t n, const int64_t *ids)
{
    IXA_REQUIRE(n >= 0 && (n == 0 || ids), kErrInvalidParam, "ids can not be nullptr.");
    const int64_t gone = remove_selected(n, ids, 0, 0, reinterpret_cast<uint32_t *>(norms_.data()));
    pad_norms();
    sync_stream(stream_);
    return gone;
}

int64_t FlatI8Index::remove_range(int64_t imin, int64_t imax)
{
    const int64_t gone = remove_selected(0, nullptr, imin, imax, reinterpret_cast<uint32_t *>(norms_.data()));
    pad_norms();
    sync_stream(stream_);
    return gone;
}

void FlatI8Index::reset()
{
    FlatBase<int8_t>::reset();
    norms_.release();
}

void FlatI8Index::search(int64_t n, const int8_t *x, int64_t k, int32_t *dist, int64_t *labels, bool on_device)
{
    search_masked(n, x, k, dist, labels, on_device, nullptr, 0);
}

// search_with_masks (FR/ascend/AscendIndexInt8Flat.h:98-99): as FlatIndex::search_with_masks
void FlatI8Index::search_with_masks(int64_t n, const int8_t *x, int64_t k, const uint8_t *mask, int32_t *dist,
                                    int64_t *labels)
{
    IXA_REQUIRE(mask, kErrInvalidParam, "mask cannot be nullptr.");
    IXA_REQUIRE(x && dist && labels, kErrInvalidParam, "x, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    const int64_t stride = (ntotal_ + 7) / 8;
    if (stride == 0) {
        search_masked(n, x, k, dist, labels, false, nullptr, 0);
        return;
    }
    const int64_t page = std::max<int64_t>(1, std::min<int64_t>(n, kMaskPageBytes / stride));
    DeviceBuffer<uint8_t> mask_dev;
    for (int64_t q0 = 0; q0 < n; q0 += page) {
        const int64_t nq = std::min(page, n - q0);
        mask_dev.upload(mask + q0 * stride, (size_t)(nq * stride), stream_);
        search_masked(nq, x + q0 * d_, k, dist + q0 * k, labels + q0 * k, false, mask_dev.data(), stride);
    }
}

void FlatI8Index::search_masked(int64_t n, const int8_t *x, int64_t k, int32_t *dist, int64_t *labels, bool on_device,
                                const uint8_t *mask_dev, int64_t mask_stride)
{
    IXA_REQUIRE(x && dist && labels, kErrInvalidParam, "x, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(k > 0 && k <= kMaxK, kErrInvalidParam, "k must be > 0 and <= %ld", (long)kMaxK);
    const int8_t *xd = x;
    if (!on_device) {
        ws_x_.upload(x, (size_t)n * d_, stream_);
        xd = ws_x_.data();
    }
    int32_t *dd = dist;
    int64_t *ld = labels;
    if (!on_device) {
        ws_dist_.resize((size_t)n * k);
        ws_labels_.resize((size_t)n * k);
        dd = ws_dist_.data();
        ld = ws_labels_.data();
    }
    ws_qn_.resize((size_t)n);
    ws_running_.resize((size_t)n * k);
    IXA_HIP(hipEventRecord(ev_[0], stream_));
    hipLaunchKernelGGL(sqnorm_rows_i8_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream_, xd, n, d_,
                       ws_qn_.data());
    const int launches = stream_select_i8(xd, n, base_.data(), ntotal_, d_, ws_qn_.data(), norms_.data(), (int)k,
                                          ws_running_.data(), ws_sel_, scratch_bytes_, stream_, mask_dev, mask_stride);
    if (mask_dev) {
        launch_drop_worst_keys_i32(ws_running_.data(), n * k, stream_);   // vectors the query leaves out
    }
    hipLaunchKernelGGL((finish_keys_kernel<int32_t, int32_t>), dim3(blocks_for(n * k)), dim3(256), 0, stream_,
                       ws_running_.data(), n * k, kMetricL2, ids_.data(), (int32_t)0x7fffffff, dd, ld);
    IXA_HIP(hipEventRecord(ev_[1], stream_));
    sync_stream(stream_);
    if (!on_device) {
        ws_dist_.download(dist, (size_t)n * k, stream_);
        ws_labels_.download(labels, (size_t)n * k, stream_);
    }
    float a = 0;
    IXA_HIP(hipEventElapsedTime(&a, ev_[0], ev_[1]));
    stats_.ms_score = 0;
    stats_.ms_select = 0;
    stats_.ms_total = a;
    stats_.score_launches = launches;
}

}  // namespace ixa
