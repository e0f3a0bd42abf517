// Host orchestration of the device-resident IVFPQ index (see ivfpq_index.h).
#include "ivfpq_index.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <mutex>
#include <numeric>
#include <random>
#include <thread>
#include <unordered_set>

#include "coarse.h"
#include "flat_i8.h"
#include "pq.h"
#include "scan.h"
#include "stream_select.h"

// Scratch of ivfpq_search_probes_device_noalloc (IvfpqIndex::search_probes_noalloc): sanitised probe lists,
// execution order and split partials of one scan launch.  Every GPU the library runs on holds its own copy
// at its own address until the process ends; in host code the name below is only a handle for
// hipGetSymbolAddress, never a device address.  (No `used` attribute: the compiler gives a static device
// variable that host code refers to a global symbol in the code object, which is what the runtime looks up;
// with the attribute the symbol stays local and the runtime aborts when the code object is loaded.)
static __device__ __align__(256) unsigned char scratch[ixa::IvfpqIndex::kNoAllocScratchBytes];

namespace ixa {

namespace {

// Address of the current device's copy of `scratch`, resolved once per device.
unsigned char *noalloc_scratch_of_current_device()
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static unsigned char *ptr[kMaxDevices] = {};
    int dev = 0;
    IXA_HIP(hipGetDevice(&dev));
    IXA_REQUIRE(dev >= 0 && dev < kMaxDevices, kErrInner, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptr[dev]) {
        void *p = nullptr;
        IXA_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        IXA_REQUIRE(p != nullptr, kErrInner, "hipGetSymbolAddress returned no address for the static scratch");
        ptr[dev] = static_cast<unsigned char *>(p);
    }
    return ptr[dev];
}

// Calls that use the static scratch of a device share it; inside one process they take turns.
std::mutex g_noalloc_mu;

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t *__restrict__ p, int n, int32_t v)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

// Parameter whitelists of the reference (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:130-140).
const int kRefDims[] = {128};
const int kRefNlists[] = {1024, 2048, 4096, 8192, 16384, 262144, 524288};
const int kRefMsubs[] = {2, 4, 8, 16, 32};

template <size_t N>
bool contains(const int (&a)[N], int64_t v)
{
    for (size_t i = 0; i < N; i++) {
        if (a[i] == v) {
            return true;
        }
    }
    return false;
}

constexpr int64_t kMaxN = 1000000000;   // MAX_N, FR/ascend/AscendIndex.h
constexpr int64_t kMaxK = 2048;         // LDS-resident selection limit of this build (reference device limit: 320)
constexpr int kMaxNprobe = 2048;        // probed lists per query (the reference's L3 operator takes 128 per tile)
constexpr int64_t kAddPage = 1 << 20;   // vectors per add page
constexpr size_t kStagedIoBytes = (size_t)1 << 20;   // host searches whose queries and results fit go through pinned staging
// Larger host searches up to this size go through the same page-locked buffer with the queries going up in two halves
// (beyond it the runtime's own path for pageable memory serves).
constexpr size_t kPipelinedIoBytes = (size_t)256 << 20;
constexpr size_t kParallelCopyBytes = (size_t)4 << 20;   // host copies of at least this much are shared by threads

// Host copies shared by up to four threads (one of them the caller's) once there is enough to move to pay for
// starting them (about 80 us for three): results that the GPU has just written into page-locked memory come out of
// DRAM, not out of the caller's cache, and a single thread moves those at 20-30 GB/s.  Thread t copies the t-th
// slice of every job.
struct CopyJob {
    void *dst;
    const void *src;
    size_t bytes;
};

void parallel_copy(std::initializer_list<CopyJob> jobs)
{
    size_t total = 0;
    for (const CopyJob &j : jobs) {
        total += j.bytes;
    }
    const unsigned hw = std::thread::hardware_concurrency();
    const int nthreads = total < kParallelCopyBytes ? 1 : (int)std::min<unsigned>(4, hw ? hw : 1);
    auto slice = [&](int t) {
        for (const CopyJob &j : jobs) {
            const size_t piece = (j.bytes / nthreads + 4095) / 4096 * 4096, off = piece * t;
            if (off < j.bytes) {
                std::memcpy(static_cast<char *>(j.dst) + off, static_cast<const char *>(j.src) + off,
                            std::min(piece, j.bytes - off));
            }
        }
    };
    std::vector<std::thread> workers;
    for (int t = 1; t < nthreads; t++) {
        workers.emplace_back(slice, t);
    }
    slice(0);
    for (auto &w : workers) {
        w.join();
    }
}
constexpr int64_t kCoarseExactMaxMacs = (int64_t)1 << 27;   // queries x centroids x dims up to which a search selects its lists exactly

// ---- arena kernels ------------------------------------------------------------------------------

// Moves lists inside one arena or from an old arena to a new one: job j copies list lists[j] (its
// src_len[j] valid entries, whole 64-slot groups) from slot src_off[j] to slot dst_off[j].  Source
// and destination ranges never overlap (a list moves to free space).  16-byte units; a list starts
// on a 64-slot boundary, so both ends are 16-byte aligned for every M.
__global__ __launch_bounds__(256) void move_lists_kernel(const uint8_t *__restrict__ src_codes,
                                                         const int64_t *__restrict__ src_ids,
                                                         const int64_t *__restrict__ src_off,
                                                         const int32_t *__restrict__ src_len,
                                                         uint8_t *__restrict__ dst_codes, int64_t *__restrict__ dst_ids,
                                                         const int64_t *__restrict__ dst_off, int M)
{
    const int j = blockIdx.x;
    const int len = src_len[j];
    if (len == 0) {
        return;
    }
    const int64_t so = src_off[j], dn = dst_off[j];
    const int64_t slots = ((int64_t)len + 63) / 64 * 64;
    const uint4 *src = reinterpret_cast<const uint4 *>(src_codes + so * M);
    uint4 *dst = reinterpret_cast<uint4 *>(dst_codes + dn * M);
    const int64_t n16 = slots * M / 16;
    for (int64_t i = threadIdx.x; i < n16; i += 256) {
        dst[i] = src[i];
    }
    for (int64_t i = threadIdx.x; i < len; i += 256) {
        dst_ids[dn + i] = src_ids[so + i];
    }
}

// list_off[lists[j]] = off[j], list_len[lists[j]] = len[j]: the device tables follow the host's for the
// lists an add touched.
__global__ __launch_bounds__(256) void update_list_tables_kernel(const int32_t *__restrict__ lists,
                                                                 const int64_t *__restrict__ off,
                                                                 const int32_t *__restrict__ len, int n,
                                                                 int64_t *__restrict__ list_off,
                                                                 int32_t *__restrict__ list_len)
{
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j < n) {
        list_off[lists[j]] = off[j];
        list_len[lists[j]] = len[j];
    }
}

// remove_ids on the device (FR/ascenddaemon/impl/IndexIVFPQ.cpp:346-506 compacts on the device too): one
// workgroup per list walks it in chunks of 256 entries; an entry whose id is in `gone` (sorted, unique) is
// dropped, the others close ranks in place keeping their order.  An entry that moves from position p to
// p2 has its code bytes re-ordered for the position-dependent layouts.  A chunk is read completely (ids
// and codes into LDS) before any of its survivors is written, and survivors only move towards the list's
// start, so in-place is safe.  Writes list_len[l], adds to *removed, and marks found[i] = 1 for every
// gone[i] it met (found may be null).
__global__ __launch_bounds__(256) void remove_ids_kernel(uint8_t *__restrict__ codes, int64_t *__restrict__ ids,
                                                         const int64_t *__restrict__ list_off,
                                                         int32_t *__restrict__ list_len, int M, int layout,
                                                         const int64_t *__restrict__ gone, int64_t n_gone,
                                                         int64_t imin, int64_t imax, uint8_t *__restrict__ found,
                                                         unsigned long long *__restrict__ removed)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    uint8_t *stage = smem_raw;                                              // 256 x M code bytes of the chunk
    int *wsum = reinterpret_cast<int *>(smem_raw + (size_t)256 * M);        // 4 wave totals
    const int l = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int len = list_len[l];
    if (len == 0) {
        return;
    }
    const int64_t off = list_off[l];
    int kept = 0;   // survivors so far (workgroup-uniform)
    for (int c0 = 0; c0 < len; c0 += 256) {
        const int p = c0 + tid;
        const bool valid = p < len;
        int64_t id = 0;
        bool drop = false;
        if (valid) {
            id = ids[off + p];
            if (gone == nullptr) {
                drop = id >= imin && id < imax;   // removal by id range
            } else {
                int64_t lo = 0, hi = n_gone;   // first element not below id
                while (lo < hi) {
                    const int64_t mid = (lo + hi) >> 1;
                    if (gone[mid] < id) {
                        lo = mid + 1;
                    } else {
                        hi = mid;
                    }
                }
                drop = lo < n_gone && gone[lo] == id;
                if (drop && found) {
                    found[lo] = 1;
                }
            }
        }
        const bool keep = valid && !drop;
        const unsigned long long m = __ballot(keep);
        const int in_wave = __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
        if (lane == 0) {
            wsum[wave] = __popcll(m);
        }
        const int chunk = len - c0 < 256 ? len - c0 : 256;
        const bool moving = kept < c0 || __syncthreads_or(valid && drop);   // an earlier drop, or one in this chunk
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            before += w < wave ? wsum[w] : 0;
            total += wsum[w];
        }
        if (moving) {
            // the chunk's code bytes are contiguous: stage them, then every survivor writes its own
            // (whole 64-slot groups in 16-byte units: a list owns its slots up to the next multiple of 64)
            const uint4 *src = reinterpret_cast<const uint4 *>(codes + (off + c0) * M);
            const int n16 = (chunk + 63) / 64 * 64 * M / 16;
            for (int i = tid; i < n16; i += 256) {
                reinterpret_cast<uint4 *>(stage)[i] = src[i];
            }
            __syncthreads();
            if (keep) {
                const int p2 = kept + before + in_wave;
                uint8_t *dst = codes + (off + p2) * M;
                const uint8_t *mine = stage + tid * M;
                for (int j = 0; j < M; j++) {
                    // byte j of the new slot holds sub-quantizer m2, which the old slot keeps at byte j1
                    int j1 = j;
                    if (layout == 1) {
                        const int m2 = (j & ~31) | ((j + p2) & 31);
                        j1 = (m2 & ~31) | ((m2 - p) & 31);
                    } else if (layout == 2) {
                        j1 = xor48_byte_of_sq(xor48_sq_of_byte(j, p2), p);
                    }
                    dst[j] = mine[j1];
                }
                ids[off + p2] = id;
            }
        }
        kept += total;
        __syncthreads();   // the staging area and the wave totals are reused by the next chunk
    }
    if (tid == 0 && kept != len) {
        list_len[l] = kept;
        atomicAdd(removed, (unsigned long long)(len - kept));
    }
}

// Places freshly encoded vectors: vector i goes to position pos[i] of list list_no[i].
// layout 1 rotates the code bytes by the position inside the list (see scan.hip).
__global__ __launch_bounds__(256) void scatter_new_kernel(int64_t n, const int32_t *__restrict__ list_no,
                                                          const int32_t *__restrict__ pos,
                                                          const uint8_t *__restrict__ codes_in,
                                                          const int64_t *__restrict__ ids_in, int64_t id_base,
                                                          const int64_t *__restrict__ new_off, int M, int layout,
                                                          uint8_t *__restrict__ codes, int64_t *__restrict__ ids)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int p = pos[i];
    const int64_t slot = new_off[list_no[i]] + p;
    const uint8_t *src = codes_in + i * M;
    uint8_t *dst = codes + slot * M;
    for (int j = 0; j < M; j++) {
        const int m = layout == 1 ? ((j & ~31) | ((j + p) & 31)) : (layout == 2 ? xor48_sq_of_byte(j, p) : j);
        dst[j] = src[m];
    }
    ids[slot] = ids_in ? ids_in[i] : id_base + i;
}

// Reads one list back in the public row-major form [len][M].
__global__ __launch_bounds__(256) void gather_list_kernel(const uint8_t *__restrict__ codes, int64_t off, int len,
                                                          int M, int layout, uint8_t *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)len * M) {
        return;
    }
    const int p = (int)(e / M), m = (int)(e % M);
    // sub-quantizer m of position p is stored at byte j with (j + p) % 32 == m % 32 inside its 32-block
    const int j = layout == 1 ? ((m & ~31) | ((m - p) & 31)) : (layout == 2 ? xor48_byte_of_sq(m, p) : m);
    out[e] = codes[(off + p) * M + j];
}

// out rows idx[i] <- rows i of the compact results (ids, and distances when given)
// out[c][t] = float( sum in float64, in list order, of x[order[i]][t] over the members i of segment c
// / their number ); segments without members keep old[c][t].  One workgroup per segment, one thread
// per component: the additions of a component happen in one fixed order.
__global__ __launch_bounds__(256) void segment_mean_kernel(const float *__restrict__ x, int d,
                                                           const int64_t *__restrict__ order,
                                                           const int64_t *__restrict__ seg,
                                                           const float *__restrict__ old, float *__restrict__ out)
{
    const int64_t c = blockIdx.x;
    const int64_t b = seg[c], e = seg[c + 1];
    for (int t = threadIdx.x; t < d; t += blockDim.x) {
        double acc = 0.0;
        for (int64_t i = b; i < e; i++) {
            acc += (double)x[order[i] * d + t];
        }
        out[c * d + t] = e > b ? (float)(acc / (double)(e - b)) : old[c * d + t];
    }
}

// ---- members of every cluster in ascending sample order, built on the device ---------------------------------
// (a stable counting sort of the samples by their cluster: counts, segment starts, members dropped into their
// segment in whatever order the hardware runs them, every segment then sorted ascending)

__global__ __launch_bounds__(256) void count_members_kernel(const int32_t *__restrict__ asg, int64_t ns,
                                                            unsigned long long *__restrict__ cnt)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < ns) {
        atomicAdd(&cnt[asg[i]], 1ull);
    }
}

// seg[c] = number of members of the clusters before c (seg[k] = all of them); cursor[c] = seg[c].  One workgroup.
__global__ __launch_bounds__(1024) void segment_starts_kernel(const unsigned long long *__restrict__ cnt, int64_t k,
                                                              int64_t *__restrict__ seg,
                                                              unsigned long long *__restrict__ cursor)
{
    __shared__ unsigned long long part[1024];
    const int64_t per = (k + 1023) / 1024, b = (int64_t)threadIdx.x * per, e = b + per < k ? b + per : k;
    unsigned long long sum = 0;
    for (int64_t c = b; c < e; c++) {
        sum += cnt[c];
    }
    part[threadIdx.x] = sum;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const unsigned long long add = threadIdx.x >= (unsigned)off ? part[threadIdx.x - off] : 0;
        __syncthreads();
        part[threadIdx.x] += add;
        __syncthreads();
    }
    unsigned long long run = part[threadIdx.x] - sum;
    for (int64_t c = b; c < e; c++) {
        seg[c] = (int64_t)run;
        cursor[c] = run;
        run += cnt[c];
    }
    if (threadIdx.x == 1023) {
        seg[k] = (int64_t)part[1023];
    }
}

__global__ __launch_bounds__(256) void place_members_kernel(const int32_t *__restrict__ asg, int64_t ns,
                                                            unsigned long long *__restrict__ cursor,
                                                            int64_t *__restrict__ order)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < ns) {
        order[atomicAdd(&cursor[asg[i]], 1ull)] = i;
    }
}

// One workgroup sorts the members of one segment ascending, in place: a bitonic network whose every exchange puts
// the smaller value at the lower position, so positions beyond the segment's end count as +infinity and are never
// touched; segments of any length (the usual one holds a few hundred members and stays in the caches).
__global__ __launch_bounds__(256) void sort_segments_kernel(int64_t *__restrict__ order, const int64_t *__restrict__ seg)
{
    int64_t *a = order + seg[blockIdx.x];
    const int64_t len = seg[blockIdx.x + 1] - seg[blockIdx.x];
    if (len < 2) {
        return;
    }
    int64_t n2 = 2;
    while (n2 < len) {
        n2 <<= 1;
    }
    for (int64_t size = 2; size <= n2; size <<= 1) {
        for (int64_t stride = size >> 1; stride > 0; stride >>= 1) {
            for (int64_t t = threadIdx.x; t < n2 / 2; t += blockDim.x) {
                // pair t of this step: the first step of a merge mirrors inside blocks of `size`, the others pair
                // positions `stride` apart
                const int64_t lo = (t / stride) * (2 * stride) + (t % stride);
                const int64_t hi = stride == size >> 1 ? (t / stride) * (2 * stride) + (2 * stride - 1 - t % stride)
                                                       : lo + stride;
                if (hi < len) {
                    const int64_t x = a[lo], y = a[hi];
                    if (x > y) {
                        a[lo] = y;
                        a[hi] = x;
                    }
                }
            }
            __threadfence_block();
            __syncthreads();
        }
    }
}

// Re-seeds empty clusters by splitting the most populated one (symmetric perturbation), in ascending order of the
// empty clusters, each split seeing the counts the earlier ones left.  One workgroup.
__global__ __launch_bounds__(1024) void split_empty_kernel(float *__restrict__ cent, unsigned long long *__restrict__ cnt,
                                                           int64_t k, int dim)
{
    __shared__ long long s_val[1024], s_idx[1024];
    const int tid = threadIdx.x;
    long long last = -1;
    while (true) {
        long long mine = INT64_MAX;
        for (long long c = last + 1 + tid; c < k; c += 1024) {
            if (cnt[c] == 0) {
                mine = c;
                break;
            }
        }
        s_idx[tid] = mine;
        __syncthreads();
        for (int off = 512; off > 0; off >>= 1) {
            if (tid < off && s_idx[tid + off] < s_idx[tid]) {
                s_idx[tid] = s_idx[tid + off];
            }
            __syncthreads();
        }
        const long long empty = s_idx[0];
        __syncthreads();
        if (empty == INT64_MAX) {
            return;
        }
        long long best = -1, at = INT64_MAX;   // the largest count, the first cluster that has it
        for (long long c = tid; c < k; c += 1024) {
            const long long v = (long long)cnt[c];
            if (v > best) {
                best = v;
                at = c;
            }
        }
        s_val[tid] = best;
        s_idx[tid] = at;
        __syncthreads();
        for (int off = 512; off > 0; off >>= 1) {
            if (tid < off) {
                const long long v = s_val[tid + off], i = s_idx[tid + off];
                if (v > s_val[tid] || (v == s_val[tid] && i < s_idx[tid])) {
                    s_val[tid] = v;
                    s_idx[tid] = i;
                }
            }
            __syncthreads();
        }
        const long long big = s_idx[0];
        __syncthreads();
        for (int t = tid; t < dim; t += 1024) {
            const float v = cent[big * dim + t];
            const float eps = (t & 1) ? 1.0f / 1024 : -1.0f / 1024;
            cent[empty * dim + t] = v * (1.0f + eps);
            cent[big * dim + t] = v * (1.0f - eps);
        }
        if (tid == 0) {
            cnt[empty] = cnt[big] / 2;
            cnt[big] -= cnt[empty];
        }
        __threadfence_block();
        __syncthreads();
        last = empty;
    }
}

// Rows scaled to unit length: the squared length summed in float64 from the first component to the last.
__global__ __launch_bounds__(256) void normalise_rows_kernel(float *__restrict__ cent, int64_t k, int dim)
{
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= k) {
        return;
    }
    double nn = 0;
    for (int t = 0; t < dim; t++) {
        nn += (double)cent[c * dim + t] * cent[c * dim + t];
    }
    nn = sqrt(nn);
    if (nn > 0) {
        for (int t = 0; t < dim; t++) {
            cent[c * dim + t] = (float)(cent[c * dim + t] / nn);
        }
    }
}

// Sub-quantizer update of PQ training: acc[m][k][t] = sum in float64, IN SAMPLE ORDER, of x[i][m*dsub + t]
// over the samples i whose code for sub-quantizer m is k; cnt[m][k] = their number.  One workgroup
// per sub-quantizer, thread k owns codeword k: tiles of 256 samples (their sub-vectors and codes) are
// staged in LDS and every thread walks the tile in order, so each sum is built in the order of the
// host loop this replaces, whatever the hardware's scheduling.
template <int DSUB>
__global__ __launch_bounds__(256) void pq_update_kernel(const float *__restrict__ x, const uint8_t *__restrict__ codes,
                                                        int64_t ns, int d, int M, double *__restrict__ acc,
                                                        long long *__restrict__ cnt)
{
    __shared__ float tile[256][DSUB + 1];
    __shared__ uint8_t tcode[256];
    const int m = blockIdx.x, k = threadIdx.x;
    double sum[DSUB];
#pragma unroll
    for (int t = 0; t < DSUB; t++) {
        sum[t] = 0.0;
    }
    long long mine = 0;
    for (int64_t i0 = 0; i0 < ns; i0 += 256) {
        const int64_t i = i0 + k;
        if (i < ns) {
            const float *src = x + i * d + m * DSUB;
#pragma unroll
            for (int t = 0; t < DSUB; t++) {
                tile[k][t] = src[t];
            }
            tcode[k] = codes[i * M + m];
        }
        __syncthreads();
        const int lim = (int)(ns - i0 < 256 ? ns - i0 : 256);
        for (int j = 0; j < lim; j++) {
            if (tcode[j] == k) {
                mine++;
#pragma unroll
                for (int t = 0; t < DSUB; t++) {
                    sum[t] += (double)tile[j][t];
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < DSUB; t++) {
        acc[((int64_t)m * 256 + k) * DSUB + t] = sum[t];
    }
    cnt[m * 256 + k] = mine;
}

template <int DSUB>
void launch_pq_update_t(const float *x, const uint8_t *codes, int64_t ns, int d, int M, double *acc, long long *cnt,
                        hipStream_t s)
{
    hipLaunchKernelGGL(pq_update_kernel<DSUB>, dim3((unsigned)M), dim3(256), 0, s, x, codes, ns, d, M, acc, cnt);
}

// false: sub-vector length not served (the caller keeps its host loop)
bool launch_pq_update(const float *x, const uint8_t *codes, int64_t ns, int d, int M, int dsub, double *acc,
                      long long *cnt, hipStream_t s)
{
    switch (dsub) {
    case 1: launch_pq_update_t<1>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 2: launch_pq_update_t<2>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 3: launch_pq_update_t<3>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 4: launch_pq_update_t<4>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 5: launch_pq_update_t<5>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 6: launch_pq_update_t<6>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 8: launch_pq_update_t<8>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 12: launch_pq_update_t<12>(x, codes, ns, d, M, acc, cnt, s); return true;
    case 16: launch_pq_update_t<16>(x, codes, ns, d, M, acc, cnt, s); return true;
    default: return false;
    }
}

__global__ __launch_bounds__(256) void scatter_rows_kernel(const int32_t *__restrict__ ids, const float *__restrict__ dist,
                                                           const int64_t *__restrict__ idx, int64_t n, int width,
                                                           int32_t *__restrict__ out_ids, float *__restrict__ out_dist)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n * width) {
        return;
    }
    const int64_t i = e / width, t = e - i * width;
    out_ids[idx[i] * width + t] = ids[e];
    if (dist) {
        out_dist[idx[i] * width + t] = dist[e];
    }
}

__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ x, const int64_t *__restrict__ idx,
                                                          int64_t n, int d, float *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n * d) {
        return;
    }
    out[e] = x[idx[e / d] * d + e % d];
}

// probe lists handed in by a caller: anything that is not a list id becomes -1 ("no list"), so that no
// later kernel indexes the list tables with it
__global__ __launch_bounds__(256) void sanitize_probes_kernel(const int32_t *__restrict__ in, int64_t n, int32_t nlist,
                                                              int32_t *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n) {
        const int32_t l = in[e];
        out[e] = (l >= 0 && l < nlist) ? l : -1;
    }
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

}  // namespace

// -------------------------------------------------------------------------------------------------

IvfpqIndex::IvfpqIndex(int d, int metric, int64_t nlist, int M, int nbits, const IvfpqConfig &cfg)
    : d_(d), M_(M), dsub_(0), metric_(metric), nlist_(nlist), cfg_(cfg)
{
    // Messages keep the reference's wording (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:510-525) so that
    // its unit tests' substring checks (FR/ut/TestAscendIndexUTIVFPQ.cpp:77-184) carry over.
    IXA_REQUIRE(metric == kMetricL2 || metric == kMetricInnerProduct, kErrInvalidParam, "Unsupported metric type");
    const bool strict = cfg.strict_reference_params != 0;
    IXA_REQUIRE(d >= 1 && d <= 4096 && (!strict || contains(kRefDims, d)), kErrInvalidParam, "Unsupported dims: %d\n",
                d);
    IXA_REQUIRE(nlist >= 1 && nlist <= (1 << 20) && (!strict || contains(kRefNlists, nlist)), kErrInvalidParam,
                "Unsupported nlists: %d\n", (int)nlist);
    IXA_REQUIRE(M >= 1 && M <= 128 && d % M == 0 && (!strict || contains(kRefMsubs, M)), kErrInvalidParam,
                "Unsupported msubs: %d\n", M);
    IXA_REQUIRE(nbits == 8, kErrInvalidParam, "Unsupported nbits: %d\n", nbits);
    dsub_ = d / M;
    if (cfg.code_layout == 1) {
        IXA_REQUIRE(M == 32 || M == 64 || M == 96, kErrInvalidParam,
                    "code layout rot32 needs msubs in {32, 64, 96}, got %d", M);
    }
    if (cfg.code_layout == 2) {
        IXA_REQUIRE(M == 48 && !cfg.lut_fp16, kErrInvalidParam, "code layout xor48 needs msubs = 48 and an fp32 LUT");
    }
    // The choice follows measurements of the scan on the benchmark shapes: 96 sub-quantizers with a half LUT
    // run 3 % faster rotated (5.21 against 5.36 ms), 48 with an fp32 LUT 11 % faster xor-rotated (4.25 against
    // 4.79 ms); 32 with an fp32 LUT run 6 % faster in plain row order (1.65 against 1.75 ms: the rotation's
    // address arithmetic costs more there than the bank conflicts it avoids), and row order sums in the
    // reference's own sequence.
    layout_ = cfg.code_layout >= 0
                  ? cfg.code_layout
                  : ((M == 64 || M == 96 || (M == 32 && cfg.lut_fp16)) ? 1 : ((M == 48 && !cfg.lut_fp16) ? 2 : 0));
    nprobe_ = (int)std::min<int64_t>(64, nlist);
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    IXA_REQUIRE(e == hipSuccess && ndev > 0, kErrIndexNotInit,
                "no HIP device available (%s): this library has no CPU path", hipGetErrorString(e));
    IXA_HIP(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    for (auto &ev : ev_) {
        IXA_HIP(hipEventCreate(&ev));
    }
    list_off_.assign((size_t)nlist_, 0);
    list_len_.assign((size_t)nlist_, 0);
    list_cap_.assign((size_t)nlist_, 0);
    sync_list_tables();
}

IvfpqIndex::~IvfpqIndex()
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

void IvfpqIndex::borrow_from(const IvfpqIndex &o)
{
    IXA_REQUIRE(d_ == o.d_ && M_ == o.M_ && metric_ == o.metric_ && nlist_ == o.nlist_, kErrInvalidParam,
                "a search view needs the shape of the index it borrows from");
    stats_pending_ = false;   // whatever they referred to is gone
    cfg_ = o.cfg_;
    layout_ = o.layout_;
    nprobe_ = o.nprobe_;
    trained_ = o.trained_;
    ntotal_ = o.ntotal_;
    max_list_len_ = o.max_list_len_;
    cmax_ = o.cmax_;
    dp_ = o.dp_;
    centroids_.borrow(o.centroids_);
    cnorm_.borrow(o.cnorm_);
    codebook_.borrow(o.codebook_);
    cbnorm_.borrow(o.cbnorm_);
    centroids_split_.borrow(o.centroids_split_);
    centroids_tiled_.borrow(o.centroids_tiled_);
    cnorm_pad_.borrow(o.cnorm_pad_);
    codes_.borrow(o.codes_);
    ids_.borrow(o.ids_);
    list_off_dev_.borrow(o.list_off_dev_);
    list_len_dev_.borrow(o.list_len_dev_);
    list_off_ = o.list_off_;
    list_len_ = o.list_len_;
    list_cap_ = o.list_cap_;
    arena_slots_ = o.arena_slots_;
    arena_used_ = o.arena_used_;
    hole_slots_ = o.hole_slots_;
}

void IvfpqIndex::set_nprobe(int nprobe)
{
    flush_stats();
    IXA_REQUIRE(nprobe >= 1, kErrInvalidParam, "nprobe must be >= 1, got %d", nprobe);
    const int clamped = (int)std::min<int64_t>(nprobe, nlist_);
    // the probe selection keeps nprobe + 16 + nprobe / 8 candidates per query in LDS
    IXA_REQUIRE(clamped <= kMaxNprobe, kErrInvalidParam, "nprobe must be <= %d, got %d", kMaxNprobe, clamped);
    nprobe_ = clamped;
}

void IvfpqIndex::check_trained() const
{
    IXA_REQUIRE(trained_, kErrIndexNotInit, "AscendIndexIVFPQ is not trained!");
}

void IvfpqIndex::sync_list_tables()
{
    max_list_len_ = list_len_.empty() ? 0 : *std::max_element(list_len_.begin(), list_len_.end());
    list_off_dev_.upload(list_off_.data(), (size_t)nlist_, stream_);
    list_len_dev_.upload(list_len_.data(), (size_t)nlist_, stream_);
    sync_stream(stream_);
}

// Everything the search keeps beside the centroids themselves (norms, bf16 splits, the splits in matrix-core order),
// from centroids_ as it stands in device memory.
void IvfpqIndex::derive_from_centroids()
{
    cnorm_.resize((size_t)nlist_);
    launch_sqnorm_rows(centroids_.data(), nlist_, d_, cnorm_.data(), stream_);
    dp_ = (int)round_up(d_, 32);
    centroids_split_.resize((size_t)nlist_ * 3 * dp_);
    launch_split_bf16x3(centroids_.data(), nlist_, d_, dp_, true, centroids_split_.data(), stream_);
    std::vector<float> cn((size_t)nlist_);
    cnorm_.download(cn.data(), cn.size(), stream_);
    cmax_ = std::sqrt(*std::max_element(cn.begin(), cn.end()));
    // The split centroids a second time, in matrix-core order, for the resident-query score kernel
    // (coarse_resident.hip), with their norms padded to whole tiles: +inf behind the last centroid, so that a
    // padding row never passes a bound; for inner product the kernel wants zeros in their place.
    centroids_tiled_.release();
    cnorm_pad_.release();
    if (resident_coarse_serves(3 * dp_)) {
        const int row_bytes = 3 * dp_ * 2;
        const int64_t padded = round_up(nlist_, kI8TileRows);
        centroids_tiled_.resize(i8_tiled_bytes(nlist_, row_bytes));
        IXA_HIP(hipMemsetAsync(centroids_tiled_.data(), 0, centroids_tiled_.bytes(), stream_));
        launch_i8_tile_rows(reinterpret_cast<const int8_t *>(centroids_split_.data()), nlist_, row_bytes,
                            reinterpret_cast<int8_t *>(centroids_tiled_.data()), 0, stream_);
        std::vector<float> pad((size_t)2 * padded, std::numeric_limits<float>::infinity());
        std::copy(cn.begin(), cn.end(), pad.begin());                       // L2: the norms
        std::fill(pad.begin() + padded, pad.begin() + padded + nlist_, 0.f);   // inner product: zeros
        cnorm_pad_.upload(pad.data(), pad.size(), stream_);
        sync_stream(stream_);   // `pad` is the source of an asynchronous copy
    }
}

// Centroid and codeword norms are produced on the device in the same left-to-right fp32 order the
// reference uses on the host (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1114-1126).
void IvfpqIndex::upload_trained(const float *centroids, const float *codebook)
{
    if (centroids) {
        centroids_.upload(centroids, (size_t)nlist_ * d_, stream_);
        derive_from_centroids();
    }
    if (codebook) {
        codebook_.upload(codebook, (size_t)M_ * 256 * dsub_, stream_);
        cbnorm_.resize((size_t)M_ * 256);
        launch_sqnorm_rows(codebook_.data(), (int64_t)M_ * 256, dsub_, cbnorm_.data(), stream_);
    }
    sync_stream(stream_);
}

void IvfpqIndex::set_trained(const float *centroids, const float *codebook)
{
    flush_stats();
    IXA_REQUIRE(centroids && codebook, kErrInvalidParam, "centroids and codebook can not be nullptr.");
    IXA_REQUIRE(ntotal_ == 0, kErrIllegalOperation, "set_trained on a non-empty index; call reset first");
    upload_trained(centroids, codebook);
    trained_ = true;
}

void IvfpqIndex::get_trained(float *centroids, float *codebook) const
{
    check_trained();
    if (centroids) {
        centroids_.download(centroids, (size_t)nlist_ * d_, stream_);
    }
    if (codebook) {
        codebook_.download(codebook, (size_t)M_ * 256 * dsub_, stream_);
    }
}

// -------------------------------------------------------------------------------------------------
// Stage 1 driver: MFMA scores into a bounded scratch, per-row selection of nout + slack candidates,
// exact refine.  Never materialises more than scratch_bytes of the n x nlist score matrix.
// Exact plan of last resort for the listed rows: canonical scores of every centroid, exact selection.
void IvfpqIndex::coarse_exact_rows(const float *x_dev, const std::vector<int64_t> &rows, int nout, int select_metric,
                                   int32_t *out_ids, float *out_dist)
{
    const int64_t m = (int64_t)rows.size();
    const int64_t per_launch = std::max<int64_t>(1, std::min<int64_t>(32768, cfg_.scratch_bytes / (4 * nlist_)));
    DeviceBuffer<int64_t> rows_dev;
    rows_dev.upload(rows.data(), rows.size(), stream_);
    DeviceBuffer<float> xsub, qn, scores, dist;
    DeviceBuffer<int32_t> idx;
    for (int64_t r0 = 0; r0 < m; r0 += per_launch) {
        const int64_t mr = std::min(per_launch, m - r0);
        xsub.resize((size_t)mr * d_);
        qn.resize((size_t)mr);
        scores.resize((size_t)mr * nlist_);
        idx.resize((size_t)mr * nout);
        hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for(mr * d_)), dim3(256), 0, stream_, x_dev,
                           rows_dev.data() + r0, mr, d_, xsub.data());
        launch_sqnorm_rows(xsub.data(), mr, d_, qn.data(), stream_);
        launch_canonical_scores(xsub.data(), mr, centroids_.data(), nlist_, d_, qn.data(), cnorm_.data(), select_metric,
                                scores.data(), nlist_, stream_);
        launch_select_rows(scores.data(), mr, nlist_, nlist_, nout, idx.data(), 0, nullptr, stream_);
        if (out_dist) {
            dist.resize((size_t)mr * nout);
            launch_gather_scores(scores.data(), nlist_, idx.data(), mr, nout, select_metric, dist.data(), stream_);
        }
        hipLaunchKernelGGL(scatter_rows_kernel, dim3(blocks_for(mr * nout)), dim3(256), 0, stream_, idx.data(),
                           out_dist ? dist.data() : nullptr, rows_dev.data() + r0, mr, nout, out_ids, out_dist);
    }
    sync_stream(stream_);   // the temporaries above are freed on return
}

// Candidate generation with matrix-core products -- bf16 x 3 (error bound below, 16 spare candidates)
// or, where that kernel does not serve the shape or is switched off, fp32 (8 spare candidates) -- then
// either the canonical re-evaluation of every candidate plus a proof that nothing outside the list can
// reach the nout-th exact score, or (set_only, bf16 x 3) the boundary-only refinement with the same
// proof.  Queries whose proof fails (near-tied centroids) are redone exactly from canonical scores of
// all centroids.
void IvfpqIndex::coarse_select(const float *x_dev, int64_t n, int nout, int select_metric, int32_t *out_ids,
                               float *out_dist, bool set_only, bool defer_check)
{
    if (n == 0) {
        return;
    }
    // A handful of queries (a search that only needs the probed SET): canonical scores of every centroid and an
    // exact selection from them, the plan coarse_exact_rows() uses for rows without proof.  Two small launches,
    // nothing to prove and no verdict for the host to read, where the matrix-core plans queue seven and a round
    // trip; worth it while the work is small (the canonical kernel reads every centroid once per query: 10M x 128
    // in 16384 lists, 32 queries: 106 us per search against 133; 20M x 768 in 32768 lists, 4 queries: 166 / 224).
    last_coarse_exact_ = cfg_.coarse_exact_small != 0 && set_only && !out_dist && n * nlist_ * d_ <= kCoarseExactMaxMacs &&
                         n <= 65535 && n * nlist_ * (int64_t)sizeof(float) <= cfg_.scratch_bytes;
    if (last_coarse_exact_) {
        last_coarse_plan_ = 0;
        last_coarse_n_ = n;
        ws_exact_.resize((size_t)n * nlist_);
        launch_canonical_scores(x_dev, n, centroids_.data(), nlist_, d_, nullptr, cnorm_.data(), select_metric,
                                ws_exact_.data(), nlist_, stream_);   // without row norms: the kernel adds them up itself
        launch_select_rows(ws_exact_.data(), n, nlist_, nlist_, nout, out_ids, 0, nullptr, stream_);
        return;
    }
    ws_qn_.resize((size_t)n);
    if (cfg_.coarse_bf16) {   // the queries' norms and their bf16 x 3 split in one launch
        ws_xsplit_.resize((size_t)n * 3 * dp_);
        launch_sqnorm_and_split_bf16x3(x_dev, n, d_, dp_, ws_qn_.data(), ws_xsplit_.data(), stream_);
    } else {
        launch_sqnorm_rows(x_dev, n, d_, ws_qn_.data(), stream_);
    }
    int ncand = (int)std::min<int64_t>(nlist_, (int64_t)nout + 16 + nout / 8);
    // flag[0] counts the queries without proof and is zero between calls: coarse_finish() clears it
    // when it was not, so the common case needs no fill in front of the kernels that append to it
    if (ws_flag_.size() < (size_t)n + 1) {   // grows only, so its first word stays what the last call left
        ws_flag_.resize((size_t)n + 1);
        flag_pending_ = true;
    }
    if (flag_pending_) {   // new memory, or a deferred verdict that was never read (a failed call in between)
        IXA_HIP(hipMemsetAsync(ws_flag_.data(), 0, sizeof(int32_t), stream_));
    }
    flag_pending_ = true;
    bool approx = false;
    last_coarse_plan_ = 0;
    last_coarse_n_ = n;
    if (cfg_.coarse_bf16) {
        ws_running_.resize((size_t)n * ncand);
        // large products: admission bound from a seed stretch, result proven by count, nothing but the seed's
        // scores written (rows without proof join the list of queries that coarse_finish() redoes exactly)
        const bool set_wanted = set_only && !out_dist && ncand > nout;   // search: only the SET of lists matters
        BoundaryRefine br{x_dev, centroids_.data(), d_, nout, cmax_, bf16x3_err_scale(select_metric),
                          select_metric == kMetricL2 ? 4.0f * 5.9604645e-8f : 0.0f, out_ids};
        const ResidentCoarse rc{reinterpret_cast<const uint16_t *>(centroids_tiled_.data()),
                                cnorm_pad_.data() + (select_metric == kMetricL2 ? 0 : round_up(nlist_, kI8TileRows)), cmax_};
        if (sampled_bound_ok_ && cfg_.coarse_sampled_bound != 0 &&
            stream_select_bf16x3_sampled(ws_xsplit_.data(), n, centroids_split_.data(), nlist_, 3 * dp_, ws_qn_.data(),
                                         cnorm_.data(), select_metric, ncand, ws_running_.data(), ws_sel_,
                                         cfg_.scratch_bytes, ws_flag_.data(), set_wanted ? &br : nullptr, stream_,
                                         centroids_tiled_.size() && cfg_.coarse_resident != 0 ? &rc : nullptr) >= 0) {
            approx = true;
            last_coarse_plan_ = 1;
            if (set_wanted) {   // the plan has written out_ids itself
                if (!defer_check) {
                    coarse_finish(x_dev, nout, select_metric, out_ids, out_dist);
                }
                return;
            }
        } else {
            approx = stream_select_bf16x3(ws_xsplit_.data(), n, centroids_split_.data(), nlist_, 3 * dp_, ws_qn_.data(),
                                          cnorm_.data(), select_metric, ncand, ws_running_.data(), ws_sel_,
                                          cfg_.scratch_bytes, stream_) >= 0;   // < 0: shape not served
        }
    }
    if (!approx) {
        ncand = (int)std::min<int64_t>(nlist_, (int64_t)nout + 8 + nout / 8);
        ws_running_.resize((size_t)n * ncand);
        stream_select_f32(x_dev, n, centroids_.data(), nlist_, d_, ws_qn_.data(), cnorm_.data(), select_metric, ncand,
                          ws_running_.data(), ws_sel_, cfg_.scratch_bytes, stream_);
    }
    // Bound on |approximate score - canonical score|, per unit of |q||c|, for one dot product.
    //   bf16 x 3: x = hi + lo + r with |lo| <= 2^-9 |x|, |r| <= 2^-18 |x|, so the three products kept miss
    //          lo.lo + r.y + x.r, at most 3 * 2^-18 sum |x_i y_i| <= 3 * 2^-18 |q||c|; bf16 x bf16 products
    //          are exact in fp32 and accumulating K = 3 dp of them in any order errs by at most
    //          K 2^-24 sum |terms|;
    //   fp32:  d rounded products summed in some order: at most (d + 1) 2^-24 sum |x_i y_i|;
    //   both:  the canonical left-to-right sum itself errs by at most (d + 1) 2^-24 sum |x_i y_i|
    //          (a few units added for the second-order terms).
    // L2 scores hold two dot products and three further roundings of numbers no larger than
    // (|q| + |c|)^2, the same on both sides up to one unit each.
    const float dots = select_metric == kMetricL2 ? 2.0f : 1.0f;
    const float u = 5.9604645e-8f;
    const float err_scale = approx ? bf16x3_err_scale(select_metric) : dots * (float)(2 * d_ + 8) * u;
    const float round_scale = select_metric == kMetricL2 ? 4.0f * u : 0.0f;
    if (approx && set_only && !out_dist && ncand > nout) {
        // search: only the SET of probed lists matters, so only the candidates the approximate scores
        // cannot decide are re-evaluated
        launch_refine_boundary(x_dev, n, centroids_.data(), d_, ws_qn_.data(), cnorm_.data(), select_metric,
                               ws_running_.data(), ncand, nout, cmax_, err_scale, round_scale, out_ids,
                               ws_flag_.data(), ncand >= nlist_, stream_);
    } else {
        float *dist = out_dist;
        if (!dist) {
            ws_exact_.resize((size_t)n * nout);
            dist = ws_exact_.data();
        }
        ws_cand_.resize((size_t)n * ncand);
        launch_keys_to_idx(ws_running_.data(), n * ncand, ws_cand_.data(), stream_);
        launch_refine(x_dev, n, centroids_.data(), d_, ws_qn_.data(), cnorm_.data(), select_metric, ws_cand_.data(),
                      ncand, nout, nout, out_ids, dist, stream_);
        if (ncand < nlist_) {   // a list that holds every centroid needs no proof
            launch_verify_superset(ws_running_.data(), ncand, dist, nout, ws_qn_.data(), cmax_, err_scale, round_scale,
                                   select_metric, n, ws_flag_.data(), stream_);
        }
    }
    if (!defer_check) {
        coarse_finish(x_dev, nout, select_metric, out_ids, out_dist);
    }
}

// Second half of coarse_select(): waits for the stream, and redoes the queries whose candidate list
// could not be proven complete from canonical scores of all centroids.  Returns how many there were.
// search() calls it after it has queued the scan behind the coarse stage, so that the common case (no
// such query) has no host round trip between the two.
// Bound on |bf16 x 3 score - canonical score| per unit of |q||c| (derivation in coarse_select()).
float IvfpqIndex::bf16x3_err_scale(int select_metric) const
{
    const float dots = select_metric == kMetricL2 ? 2.0f : 1.0f;
    return dots * (3.0f / 262144.0f + (float)(3 * dp_ + d_ + 8) * 5.9604645e-8f);
}

int IvfpqIndex::coarse_finish(const float *x_dev, int nout, int select_metric, int32_t *out_ids, float *out_dist,
                              std::vector<int32_t> *redone)
{
    if (last_coarse_exact_) {
        return 0;   // exact by construction: no list of rows without proof exists
    }
    int32_t nfail = 0;
    ws_flag_.download(&nfail, 1, stream_);
    if (nfail == 0) {
        flag_pending_ = false;
        return 0;
    }
    last_coarse_reruns_ += nfail;
    if (last_coarse_plan_ == 1 && (int64_t)nfail * 16 > last_coarse_n_) {
        // the seed stretch does not represent this index's centroids (they come in some order): every
        // such query costs an exact rerun, so the plan that writes the score matrix is the cheaper one
        sampled_bound_ok_ = false;
    }
    std::vector<int32_t> rows32((size_t)nfail);
    IXA_HIP(hipMemcpyAsync(rows32.data(), ws_flag_.data() + 1, (size_t)nfail * 4, hipMemcpyDeviceToHost, stream_));
    IXA_HIP(hipMemsetAsync(ws_flag_.data(), 0, sizeof(int32_t), stream_));
    sync_stream(stream_);
    flag_pending_ = false;
    std::sort(rows32.begin(), rows32.end());   // the order of the appends is not deterministic
    coarse_exact_rows(x_dev, std::vector<int64_t>(rows32.begin(), rows32.end()), nout, select_metric, out_ids, out_dist);
    if (redone) {
        *redone = std::move(rows32);
    }
    return nfail;
}

void IvfpqIndex::assign(int64_t n, const float *x, int64_t *out, bool on_device)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(x && out, kErrInvalidParam, "x can not be nullptr.");
    IXA_REQUIRE(n >= 0 && n < kMaxN, kErrInvalidParam, "n must be >= 0 and < %ld", (long)kMaxN);
    std::vector<int32_t> tmp;
    for (int64_t p0 = 0; p0 < n; p0 += kAddPage) {
        const int64_t np = std::min(kAddPage, n - p0);
        const float *xd = x + p0 * d_;
        if (!on_device) {
            ws_x_.upload(x + p0 * d_, (size_t)np * d_, stream_);
            xd = ws_x_.data();
        }
        ws_probes_.resize((size_t)np);
        coarse_select(xd, np, 1, kMetricL2, ws_probes_.data(), nullptr);
        tmp.resize((size_t)np);
        ws_probes_.download(tmp.data(), (size_t)np, stream_);
        for (int64_t i = 0; i < np; i++) {
            out[p0 + i] = tmp[(size_t)i];
        }
    }
}

void IvfpqIndex::coarse_probe(int64_t n, const float *x, int64_t *out_ids, float *out_dist, bool on_device)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(x && out_ids, kErrInvalidParam, "x can not be nullptr.");
    const float *xd = x;
    if (!on_device) {
        ws_x_.upload(x, (size_t)n * d_, stream_);
        xd = ws_x_.data();
    }
    ws_probes_.resize((size_t)n * nprobe_);
    ws_dist_.resize((size_t)n * nprobe_);
    coarse_select(xd, n, nprobe_, metric_, ws_probes_.data(), ws_dist_.data());
    std::vector<int32_t> tmp((size_t)n * nprobe_);
    ws_probes_.download(tmp.data(), tmp.size(), stream_);
    for (size_t i = 0; i < tmp.size(); i++) {
        out_ids[i] = tmp[i];
    }
    if (out_dist) {
        ws_dist_.download(out_dist, (size_t)n * nprobe_, stream_);
    }
}

void IvfpqIndex::encode(int64_t n, const float *x, uint8_t *codes, bool on_device)
{
    check_trained();
    IXA_REQUIRE(x && codes, kErrInvalidParam, "x can not be nullptr.");
    DeviceBuffer<uint8_t> cd;
    for (int64_t p0 = 0; p0 < n; p0 += kAddPage) {
        const int64_t np = std::min(kAddPage, n - p0);
        const float *xd = x + p0 * d_;
        if (!on_device) {
            ws_x_.upload(x + p0 * d_, (size_t)np * d_, stream_);
            xd = ws_x_.data();
        }
        cd.resize((size_t)np * M_);
        launch_pq_encode(xd, np, d_, M_, codebook_.data(), cd.data(), stream_);
        cd.download(codes + p0 * M_, (size_t)np * M_, stream_);
    }
}

// -------------------------------------------------------------------------------------------------
// add: coarse assignment (always L2, as the reference's add path: AscendIndexIVFPQImpl.cpp:603-672,
// 701), PQ encode of the raw vector (:674-692, 879-921), then append to the lists in input order
// (:715-805; ids default to ntotal + i, FR/ascend/impl/AscendIndexImpl.h:59-83).
void IvfpqIndex::add(int64_t n, const float *x, const int64_t *ids, bool on_device)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(x, kErrInvalidParam, "x can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(ntotal_ + n < ((int64_t)1 << 32) - 64 * nlist_, kErrInvalidParam,
                "index would exceed the 32-bit slot space");
    // (workspaces of the add path live in the index: a small add must not pay for allocations)
    DeviceBuffer<int32_t> &list_no = ws_add_lists_;
    DeviceBuffer<uint8_t> &codes = ws_add_codes_;
    DeviceBuffer<int64_t> &ids_dev = ws_add_ids_;
    for (int64_t p0 = 0; p0 < n; p0 += kAddPage) {
        const int64_t np = std::min(kAddPage, n - p0);
        const float *xd = x + p0 * d_;
        if (!on_device) {
            ws_x_.upload(x + p0 * d_, (size_t)np * d_, stream_);
            xd = ws_x_.data();
        }
        const int64_t *idd = nullptr;
        if (ids) {
            if (on_device) {
                idd = ids + p0;
            } else {
                ids_dev.upload(ids + p0, (size_t)np, stream_);
                idd = ids_dev.data();
            }
        }
        list_no.resize((size_t)np);
        // the verdict of the assignment's proof is read together with the assignments (one wait, not two)
        coarse_select(xd, np, 1, kMetricL2, list_no.data(), nullptr, false, true);
        codes.resize((size_t)np * M_);
        launch_pq_encode(xd, np, d_, M_, codebook_.data(), codes.data(), stream_);
        append(np, list_no.data(), codes.data(), idd, xd);
    }
}

void IvfpqIndex::add_codes(int64_t list, int64_t n, const uint8_t *codes, const int64_t *ids)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(list >= 0 && list < nlist_, kErrInvalidParam, "the listId is %ld, out of numLists(%ld)", (long)list,
                (long)nlist_);
    IXA_REQUIRE(n >= 0 && (n == 0 || (codes && ids)), kErrInvalidParam, "codes and ids can not be nullptr.");
    if (n == 0) {
        return;
    }
    std::vector<int32_t> ln((size_t)n, (int32_t)list);
    DeviceBuffer<int32_t> list_no;
    DeviceBuffer<uint8_t> cd;
    DeviceBuffer<int64_t> idd;
    list_no.upload(ln.data(), (size_t)n, stream_);
    cd.upload(codes, (size_t)n * M_, stream_);
    idd.upload(ids, (size_t)n, stream_);
    append(n, list_no.data(), cd.data(), idd.data());
}

void IvfpqIndex::add_codes_bulk(int64_t n, const int32_t *list_no, const uint8_t *codes, const int64_t *ids)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(n >= 0 && (n == 0 || (list_no && codes && ids)), kErrInvalidParam, "codes and ids can not be nullptr.");
    if (n == 0) {
        return;
    }
    DeviceBuffer<int32_t> ln;
    DeviceBuffer<uint8_t> cd;
    DeviceBuffer<int64_t> idd;
    ln.upload(list_no, (size_t)n, stream_);
    cd.upload(codes, (size_t)n * M_, stream_);
    idd.upload(ids, (size_t)n, stream_);
    append(n, ln.data(), cd.data(), idd.data());
}

// Appends n encoded vectors to their lists, positions inside a list following input order.  Lists have
// slack: a list whose new length fits its capacity is extended in place; one that does not moves to free
// space at the end of the arena with half as much room again (a list that is new gets what it needs); when
// the arena itself is full, a new one (at least half as large again) takes every list in id order, which
// also reclaims the holes that moved lists left.  An add therefore touches the lists it extends and, now
// and then, pays for a compaction that its predecessors' growth amortises
// (FR/ascenddaemon/impl/IndexIVFPQ.cpp:210-235 appends to per-list device vectors in the same way).  Host
// tables change only after the device work has succeeded.
void IvfpqIndex::append(int64_t n, const int32_t *list_no_dev, const uint8_t *codes_dev, const int64_t *ids_dev,
                        const float *assigned_from)
{
    // assigned_from: the vectors whose coarse assignment (queued with a deferred verdict) produced list_no_dev
    int32_t *stage = static_cast<int32_t *>(add_stage_.reserve(((size_t)n + 1) * 4));
    int32_t *list_no = stage + 1;
    stage[0] = 0;
    if (assigned_from) {
        IXA_HIP(hipMemcpyAsync(stage, ws_flag_.data(), 4, hipMemcpyDeviceToHost, stream_));
    }
    IXA_HIP(hipMemcpyAsync(list_no, list_no_dev, (size_t)n * 4, hipMemcpyDeviceToHost, stream_));
    sync_stream(stream_);
    if (assigned_from) {
        if (stage[0] != 0) {
            // some assignments could not be proven: they are redone exactly, and read again
            coarse_finish(assigned_from, 1, kMetricL2, const_cast<int32_t *>(list_no_dev), nullptr);
            IXA_HIP(hipMemcpyAsync(list_no, list_no_dev, (size_t)n * 4, hipMemcpyDeviceToHost, stream_));
            sync_stream(stream_);
        } else {
            flag_pending_ = false;
        }
    }
    std::vector<int32_t> &pos = add_pos_;
    pos.resize((size_t)n);
    // positions of the new vectors, and the lists they touch (in order of first appearance)
    std::vector<int32_t> touched, new_len_t;
    if (touch_mark_.size() != (size_t)nlist_) {
        touch_mark_.assign((size_t)nlist_, -1);
    }
    for (int64_t i = 0; i < n; i++) {
        const int32_t l = list_no[i];
        if (!(l >= 0 && l < nlist_)) {
            for (int32_t t : touched) {
                touch_mark_[(size_t)t] = -1;
            }
            fail(kErrInner, "coarse assignment produced list %d", l);
        }
        int32_t &slot = touch_mark_[(size_t)l];
        if (slot < 0) {
            slot = (int32_t)touched.size();
            touched.push_back(l);
            new_len_t.push_back(list_len_[(size_t)l]);
        }
        pos[(size_t)i] = new_len_t[(size_t)slot]++;
    }
    for (int32_t t : touched) {
        touch_mark_[(size_t)t] = -1;
    }
    // lists that outgrow their capacity
    std::vector<int32_t> grow;          // indices into `touched`
    std::vector<int64_t> new_cap_t(touched.size());
    int64_t grow_slots = 0, freed_slots = 0;
    for (size_t t = 0; t < touched.size(); t++) {
        const int32_t l = touched[t];
        new_cap_t[t] = list_cap_[(size_t)l];
        if (new_len_t[t] > list_cap_[(size_t)l]) {
            const int64_t want = list_cap_[(size_t)l] == 0 ? new_len_t[t] : (int64_t)new_len_t[t] + new_len_t[t] / 2;
            new_cap_t[t] = round_up(want, 64);
            grow.push_back((int32_t)t);
            grow_slots += new_cap_t[t];
            freed_slots += list_cap_[(size_t)l];
        }
    }
    IXA_REQUIRE(arena_used_ - hole_slots_ - freed_slots + grow_slots < ((int64_t)1 << 32) - 1, kErrInvalidParam,
                "index exceeds the 32-bit slot space");
    if (arena_used_ + grow_slots > arena_slots_ || (hole_slots_ + freed_slots) * 2 > arena_used_ + grow_slots) {
        // the arena is full, or half of it would be holes: a new one takes every list in id order, the growing
        // lists with their new capacities, and leaves half as much room again for lists that move later
        std::vector<int32_t> cap_all(list_cap_);
        for (size_t t = 0; t < touched.size(); t++) {
            cap_all[(size_t)touched[t]] = (int32_t)new_cap_t[t];
        }
        const int64_t live = arena_used_ - hole_slots_ - freed_slots + grow_slots;
        relayout(cap_all, live + live / 2);
        grow.clear();
        freed_slots = 0;
    }
    std::vector<int64_t> new_off_t(touched.size());
    for (size_t t = 0; t < touched.size(); t++) {
        new_off_t[t] = list_off_[(size_t)touched[t]];
    }
    int64_t new_used = arena_used_;
    // everything the kernels below read goes up in ONE copy of 64-bit words:
    //   [move jobs: src, dst, len of each growing list][touched lists: list, new first slot, new length][positions]
    const size_t ng = grow.size(), nt = touched.size();
    const size_t pack_words = 3 * ng + 3 * nt + ((size_t)n + 1) / 2;
    int64_t *pack = static_cast<int64_t *>(add_pack_.reserve(pack_words * 8));
    for (size_t g = 0; g < ng; g++) {
        const size_t t = (size_t)grow[g];
        const int32_t l = touched[t];
        pack[g] = list_off_[(size_t)l];
        pack[ng + g] = new_used;
        reinterpret_cast<int32_t *>(pack + 2 * ng)[g] = list_len_[(size_t)l];
        new_off_t[t] = new_used;
        new_used += new_cap_t[t];
    }
    int64_t *pt = pack + 3 * ng;
    for (size_t t = 0; t < nt; t++) {
        pt[t] = new_off_t[t];
        reinterpret_cast<int32_t *>(pt + nt)[t] = touched[t];
        reinterpret_cast<int32_t *>(pt + 2 * nt)[t] = new_len_t[t];
    }
    std::memcpy(pt + 3 * nt, pos.data(), (size_t)n * 4);
    try {
        ws_add_pack_.upload(pack, pack_words, stream_);
        const int64_t *dp = ws_add_pack_.data();
        if (ng > 0) {
            // the lists that outgrew their place move to the end of the used part
            hipLaunchKernelGGL(move_lists_kernel, dim3((unsigned)ng), dim3(256), 0, stream_, codes_.data(), ids_.data(),
                               dp, reinterpret_cast<const int32_t *>(dp + 2 * ng), codes_.data(), ids_.data(), dp + ng,
                               M_);
        }
        // the device tables follow for the touched lists, then the new vectors are placed by them
        const int64_t *dt = dp + 3 * ng;
        hipLaunchKernelGGL(update_list_tables_kernel, dim3(blocks_for((int64_t)nt)), dim3(256), 0, stream_,
                           reinterpret_cast<const int32_t *>(dt + nt), dt, reinterpret_cast<const int32_t *>(dt + 2 * nt),
                           (int)nt, list_off_dev_.data(), list_len_dev_.data());
        hipLaunchKernelGGL(scatter_new_kernel, dim3(blocks_for(n)), dim3(256), 0, stream_, n, list_no_dev,
                           reinterpret_cast<const int32_t *>(dt + 3 * nt), codes_dev, ids_dev, ntotal_,
                           list_off_dev_.data(), M_, layout_, codes_.data(), ids_.data());
        sync_stream(stream_);
    } catch (...) {
        sync_list_tables();   // the device tables go back to what the host says (the lists themselves are untouched)
        throw;
    }
    // success: the host's view follows
    for (size_t t = 0; t < touched.size(); t++) {
        const int32_t l = touched[t];
        list_off_[(size_t)l] = new_off_t[t];
        list_len_[(size_t)l] = new_len_t[t];
        list_cap_[(size_t)l] = (int32_t)new_cap_t[t];
        max_list_len_ = std::max(max_list_len_, new_len_t[t]);
    }
    arena_used_ = new_used;
    hole_slots_ += freed_slots;
    ntotal_ += n;
}

// A new arena of at least min_slots slots takes every list in id order, list l with cap[l] slots (>= its
// length rounded up to 64).  The old arena is released only after the new one is complete, so a failure
// (no memory for the second copy) leaves the index as it was.
void IvfpqIndex::relayout(const std::vector<int32_t> &cap, int64_t min_slots)
{
    std::vector<int64_t> off((size_t)nlist_);
    int64_t at = 0;
    for (int64_t l = 0; l < nlist_; l++) {
        off[(size_t)l] = at;
        at += cap[(size_t)l];
    }
    int64_t slots = round_up(std::max<int64_t>({at, min_slots, 1024}), 64);
    slots = std::min<int64_t>(slots, ((int64_t)1 << 32) - 64);
    IXA_REQUIRE(slots >= at, kErrInvalidParam, "index exceeds the 32-bit slot space");
    DeviceBuffer<uint8_t> new_codes((size_t)slots * M_);
    DeviceBuffer<int64_t> new_ids((size_t)slots);
    DeviceBuffer<int64_t> off_dev;
    IXA_HIP(hipMemsetAsync(new_codes.data(), 0, new_codes.bytes(), stream_));
    IXA_HIP(hipMemsetAsync(new_ids.data(), 0xff, new_ids.bytes(), stream_));
    off_dev.upload(off.data(), (size_t)nlist_, stream_);
    if (ntotal_ > 0) {
        hipLaunchKernelGGL(move_lists_kernel, dim3((unsigned)nlist_), dim3(256), 0, stream_, codes_.data(), ids_.data(),
                           list_off_dev_.data(), list_len_dev_.data(), new_codes.data(), new_ids.data(), off_dev.data(),
                           M_);
    }
    sync_stream(stream_);
    codes_ = std::move(new_codes);
    ids_ = std::move(new_ids);
    list_off_ = std::move(off);
    list_cap_ = cap;
    arena_slots_ = slots;
    arena_used_ = at;
    hole_slots_ = 0;
    list_off_dev_.upload(list_off_.data(), (size_t)nlist_, stream_);
    sync_stream(stream_);
}

// AscendIndexIVF::reserveMemory(numVecs) (FR/ascend/AscendIndexIVF.h): room for num_vecs more vectors before
// the arena has to be replaced (spread over the lists in proportion to nothing: lists still move inside the
// arena as they grow; what is reserved is the arena itself).
void IvfpqIndex::reserve_memory(int64_t num_vecs)
{
    flush_stats();
    IXA_REQUIRE(num_vecs >= 0 && num_vecs < kMaxN, kErrInvalidParam, "numVecs must be >= 0 and < %ld", (long)kMaxN);
    // every list may round its share up to a multiple of 64 and move once with half as much room again
    const int64_t want = arena_used_ + num_vecs + num_vecs / 2 + 64 * nlist_;
    if (want > arena_slots_) {
        relayout(list_cap_, std::min<int64_t>(want, ((int64_t)1 << 32) - 64));
    }
}

// AscendIndexIVF::reclaimMemory() (FR/ascend/AscendIndexIVF.h): gives back what the lists do not use; returns
// the bytes released.
int64_t IvfpqIndex::reclaim_memory()
{
    flush_stats();
    const int64_t before = arena_slots_;
    std::vector<int32_t> cap((size_t)nlist_);
    int64_t need = 0;
    for (int64_t l = 0; l < nlist_; l++) {
        cap[(size_t)l] = (int32_t)round_up(list_len_[(size_t)l], 64);
        need += cap[(size_t)l];
    }
    if (ntotal_ == 0) {
        reset();
        return before * (M_ + 8);
    }
    if (round_up(std::max<int64_t>(need, 1024), 64) >= before) {
        return 0;
    }
    relayout(cap, 0);
    return (before - arena_slots_) * (M_ + 8);
}

int64_t IvfpqIndex::list_length(int64_t list) const
{
    IXA_REQUIRE(list >= 0 && list < nlist_, kErrInvalidParam, "the listId is %ld, out of numLists(%ld)", (long)list,
                (long)nlist_);
    return list_len_[(size_t)list];
}

void IvfpqIndex::get_list(int64_t list, uint8_t *codes, int64_t *ids) const
{
    const int64_t len = list_length(list);
    if (len == 0) {
        return;
    }
    const int64_t off = list_off_[(size_t)list];
    if (codes) {
        DeviceBuffer<uint8_t> tmp((size_t)len * M_);
        hipLaunchKernelGGL(gather_list_kernel, dim3(blocks_for(len * M_)), dim3(256), 0, stream_, codes_.data(), off,
                           (int)len, M_, layout_, tmp.data());
        tmp.download(codes, (size_t)len * M_, stream_);
    }
    if (ids) {
        IXA_HIP(hipMemcpyAsync(ids, ids_.data() + off, (size_t)len * 8, hipMemcpyDeviceToHost, stream_));
        sync_stream(stream_);
    }
}

// remove_ids: every list is filtered in place on the device, keeping the order of the survivors
// (FR/ascenddaemon/impl/IndexIVFPQ.cpp:346-506).  The ids go up sorted; one workgroup per list looks its
// entries up by bisection and compacts.  `found`, when given, receives for every entry of the SORTED
// UNIQUE id list whether the index held it.
int64_t IvfpqIndex::remove_sorted_ids(const std::vector<int64_t> &gone, std::vector<uint8_t> *found)
{
    return remove_selected(&gone, 0, 0, found);
}

// gone != nullptr: the sorted unique ids to remove; otherwise the ids in [imin, imax) leave.
int64_t IvfpqIndex::remove_selected(const std::vector<int64_t> *gone_ids, int64_t imin, int64_t imax,
                                    std::vector<uint8_t> *found)
{
    static const std::vector<int64_t> none;
    const std::vector<int64_t> &gone = gone_ids ? *gone_ids : none;
    if ((gone_ids ? gone.empty() : imin >= imax) || ntotal_ == 0) {
        if (found) {
            found->assign(gone.size(), 0);
        }
        return 0;
    }
    DeviceBuffer<int64_t> gone_dev;
    DeviceBuffer<uint8_t> found_dev;
    DeviceBuffer<unsigned long long> removed_dev(1);
    if (gone_ids) {
        gone_dev.upload(gone.data(), gone.size(), stream_);
    }
    if (found) {
        found_dev.resize(gone.size());
        IXA_HIP(hipMemsetAsync(found_dev.data(), 0, found_dev.bytes(), stream_));
    }
    IXA_HIP(hipMemsetAsync(removed_dev.data(), 0, 8, stream_));
    const size_t smem = (size_t)256 * M_ + 64;
    hipLaunchKernelGGL(remove_ids_kernel, dim3((unsigned)nlist_), dim3(256), smem, stream_, codes_.data(), ids_.data(),
                       list_off_dev_.data(), list_len_dev_.data(), M_, layout_,
                       gone_ids ? gone_dev.data() : (const int64_t *)nullptr, (int64_t)gone.size(), imin, imax,
                       found ? found_dev.data() : nullptr, removed_dev.data());
    unsigned long long removed = 0;
    removed_dev.download(&removed, 1, stream_);
    if (found) {
        found->resize(gone.size());
        found_dev.download(found->data(), gone.size(), stream_);
    }
    if (removed > 0) {
        list_len_dev_.download(list_len_.data(), (size_t)nlist_, stream_);
        max_list_len_ = *std::max_element(list_len_.begin(), list_len_.end());
        ntotal_ -= (int64_t)removed;
    }
    return (int64_t)removed;
}

int64_t IvfpqIndex::remove_ids(int64_t n, const int64_t *ids)
{
    flush_stats();
    IXA_REQUIRE(n >= 0 && (n == 0 || ids), kErrInvalidParam, "ids can not be nullptr.");
    if (n == 0 || ntotal_ == 0) {
        return 0;
    }
    std::vector<int64_t> gone(ids, ids + n);
    std::sort(gone.begin(), gone.end());
    gone.erase(std::unique(gone.begin(), gone.end()), gone.end());
    return remove_sorted_ids(gone, nullptr);
}

// remove_ids(IDSelectorRange) (FR/ascend/impl/AscendIndexIVFImpl.cpp:432-440): the ids in [imin, imax) leave
int64_t IvfpqIndex::remove_range(int64_t imin, int64_t imax)
{
    flush_stats();
    return remove_selected(nullptr, imin, imax, nullptr);
}

// update (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:540-601): ids that exist are deleted and re-added with
// their new vectors (they move to the end of their new list); ids that do not exist are returned.
std::vector<int64_t> IvfpqIndex::update(int64_t n, const float *x, const int64_t *ids)
{
    flush_stats();
    check_trained();
    IXA_REQUIRE(x, kErrInvalidParam, "vector list is nullptr!");
    IXA_REQUIRE(ids, kErrInvalidParam, "vector ID list is nullptr!");
    IXA_REQUIRE(n > 0, kErrInvalidParam, "update vector number must be greater than 0!");
    std::vector<int64_t> gone(ids, ids + n);
    std::sort(gone.begin(), gone.end());
    gone.erase(std::unique(gone.begin(), gone.end()), gone.end());
    std::vector<uint8_t> found;
    remove_sorted_ids(gone, &found);   // the removal itself tells which ids the index held
    std::vector<int64_t> missing, exist_ids;
    std::vector<float> exist_x;
    for (int64_t i = 0; i < n; i++) {
        const size_t at = (size_t)(std::lower_bound(gone.begin(), gone.end(), ids[i]) - gone.begin());
        if (found[at]) {
            exist_ids.push_back(ids[i]);
            exist_x.insert(exist_x.end(), x + i * d_, x + (i + 1) * d_);
        } else {
            missing.push_back(ids[i]);
        }
    }
    if (!exist_ids.empty()) {
        add((int64_t)exist_ids.size(), exist_x.data(), exist_ids.data(), false);
    }
    return missing;
}

// reset keeps the trained quantizers and drops every list (FR/ascend/AscendIndexIVF.h: reset()).
void IvfpqIndex::reset()
{
    flush_stats();
    sync_stream(stream_);
    codes_.release();
    ids_.release();
    list_off_.assign((size_t)nlist_, 0);
    list_len_.assign((size_t)nlist_, 0);
    list_cap_.assign((size_t)nlist_, 0);
    arena_slots_ = arena_used_ = hole_slots_ = 0;
    ntotal_ = 0;
    sync_list_tables();
}

// Workgroups per query of the scan.  Small batches are split over several workgroups per query.  Every workgroup
// builds the query's whole LUT, so more of them cost more than they balance unless each keeps thousands of codes
// to scan: up to eight per query and about 384 in all when a query's lists hold few codes (measured at nlist
// 16384, nprobe 64, 39000 codes per query: 8 queries 0.31 -> 0.16 ms and 64 queries 0.33 -> 0.17 ms against a
// rule that aimed at 2048 workgroups), up to 64 per query and about 1024 in all while a workgroup keeps 4096
// codes or more on average (nlist 1024 on 10M vectors, nprobe 32: 312000 codes per query; a single query is
// bound by the latency of one wave's loads, and 8 workgroups leave 98 % of the GPU idle).  From about 400
// queries on one workgroup per query is best.  The slices are merged by radix selection, whose cost does not
// grow with their number.
int IvfpqIndex::scan_nsplit(int64_t n, int nprobe, int64_t k, int64_t codes_per_query)
{
    (void)k;
    const int64_t cap = std::max<int64_t>(8, std::min<int64_t>(64, codes_per_query / 4096));
    const int64_t target = cap > 8 ? 1024 : 384;
    const int64_t nsplit = std::max<int64_t>(1, std::min<int64_t>(cap, (target + n / 2) / n));
    return (int)std::min<int64_t>(nsplit, nprobe);
}

// Parameters of the fused LUT + scan + top-k launch for `n` queries and their probe lists.  With `ext` the
// launch's scratch (split partials, execution order) lies in memory the caller provides and nothing is
// allocated here.
ScanParams IvfpqIndex::scan_params(const float *xd, int64_t n, const int32_t *probes, int nprobe, int64_t k, float *dd,
                                   int64_t *ld, const ScanScratch *ext)
{
    ScanParams p{};
    p.queries = xd;
    p.probes = probes;
    p.nprobe = nprobe;
    p.codebook = codebook_.data();
    p.cb_norms = cbnorm_.data();
    p.d = d_;
    p.M = M_;
    p.dsub = dsub_;
    p.metric = metric_;
    p.lut_fp16 = cfg_.lut_fp16;
    p.codes = codes_.data();
    p.ids = ids_.data();
    p.list_off = list_off_dev_.data();
    p.list_len = list_len_dev_.data();
    p.nlist = nlist_;
    p.code_layout = layout_;
    p.k = (int)k;
    const int nsplit = scan_nsplit(n, nprobe, k, nlist_ > 0 ? ntotal_ / nlist_ * nprobe : 0);
    p.nsplit = nsplit;
    if (nsplit > 1) {
        if (ext) {
            p.partial = ext->partial;
        } else {
            ws_partial_.resize((size_t)n * nsplit * k);
            p.partial = ws_partial_.data();
        }
    }
    p.out_dist = dd;
    p.out_labels = ld;
    // Few workgroups (at most eight rounds of a full GPU), each with enough work that a late heavy one
    // shows: start the heaviest queries first.  Measured on 100M Zipf-skewed vectors, 1024 queries, nprobe 256: scan 5.4 -> 4.95 ms;
    // no effect on 10000 queries over even lists.
    p.order = nullptr;
    const int64_t codes_per_group = nlist_ > 0 ? ntotal_ / nlist_ * nprobe / nsplit : 0;   // average work of a workgroup
    // order | class of every query, and histogram (zero between calls) | cursors of the counting sort
    int32_t *order = ext ? ext->order : nullptr, *hist = ext ? ext->hist : nullptr;
    auto own_order_buffers = [&]() {
        if (ext) {
            return;
        }
        ws_order_.resize((size_t)n * 2);
        if (ws_order_hist_.size() == 0) {
            ws_order_hist_.resize(2 * 1024);
            IXA_HIP(hipMemsetAsync(ws_order_hist_.data(), 0, ws_order_hist_.bytes(), stream_));
        }
        order = ws_order_.data();
        hist = ws_order_hist_.data();
    };
    if (n * nsplit <= 8192 && n >= 64 && codes_per_group >= 16384) {
        own_order_buffers();
        launch_order_by_work(probes, n, nprobe, list_len_dev_.data(), nlist_, (long long)nprobe * max_list_len_, order + n, hist,
                             hist + 1024, order, stream_);
        p.order = order;
    }
    // Large batches, one workgroup per query: queries that probe the same lists are made neighbours in the
    // execution order and every XCD takes a contiguous chunk of it, so that lists shared by neighbours are
    // fetched into that XCD's L2 once.
    p.xcd_chunks = 0;
    const bool by_locality = cfg_.scan_locality < 0 ? n >= 2048 : cfg_.scan_locality > 0;
    if (!p.order && nsplit == 1 && n >= 16 && by_locality) {
        own_order_buffers();
        launch_order_by_locality(probes, n, nprobe, order + n, hist, hist + 1024, order, stream_);
        p.order = order;
        p.xcd_chunks = 1;
    }
    return p;
}

// Stages 2-4 on caller-supplied probe lists (AscendcIvfpqSearchDistanceL2 + TopkIvfpqL3 of the
// reference, FR/ascenddaemon/impl/IndexIVFPQ.cpp:2162-2347, with the LUT built inside the launch):
// probes[n][nprobe] list ids on the device, -1 = no list.
void IvfpqIndex::search_probes(int64_t n, const float *x_dev, const int32_t *probes_dev, int nprobe, int64_t k,
                               float *dist_dev, int64_t *labels_dev)
{
    check_trained();
    IXA_REQUIRE(x_dev && probes_dev && dist_dev && labels_dev, kErrInvalidParam,
                "x, probes, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(k > 0 && k <= kMaxK, kErrInvalidParam, "k must be > 0 and <= %ld", (long)kMaxK);
    IXA_REQUIRE(nprobe > 0 && nprobe <= nlist_, kErrInvalidParam, "nprobe must be > 0 and <= nlist");
    flush_stats();
    ws_probes_.resize((size_t)n * nprobe);
    hipLaunchKernelGGL(sanitize_probes_kernel, dim3(blocks_for(n * nprobe)), dim3(256), 0, stream_, probes_dev,
                       n * nprobe, (int32_t)nlist_, ws_probes_.data());
    ScanParams p = scan_params(x_dev, n, ws_probes_.data(), nprobe, k, dist_dev, labels_dev);
    launch_scan(p, n, stream_);
    sync_stream(stream_);
    // the plan of this launch; no stage timings are taken here
    stats_ = SearchStats{};
    stats_.nsplit = p.nsplit;
    stats_.scan_launches = p.nsplit > 1 ? 2 : 1;
    stats_.ordered = p.order ? (p.xcd_chunks ? 2 : 1) : 0;   // 1 = heaviest first, 2 = by locality
    plan_scan(p);
    stats_.scan_waves = p.waves;
    stats_.shared_pool = p.shared_pool;
}

// The same call with nothing allocated, for callers that cannot call hipMalloc (tight serving loops, harnesses
// that forbid allocation; it launches on the index's own stream and waits for the results, so it is not a call
// to make under stream capture): the sanitised probe lists, the execution order and the split partials lie in the static
// device scratch, laid out as [histogram | cursors: 8 KB][order | class: 8 n][probes: 4 n nprobe]
// [partials: 8 n nsplit k], each part rounded up to 256 bytes.
void IvfpqIndex::search_probes_noalloc(int64_t n, const float *x_dev, const int32_t *probes_dev, int nprobe, int64_t k,
                                       float *dist_dev, int64_t *labels_dev)
{
    check_trained();
    IXA_REQUIRE(x_dev && probes_dev && dist_dev && labels_dev, kErrInvalidParam,
                "x, probes, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(k > 0 && k <= kMaxK, kErrInvalidParam, "k must be > 0 and <= %ld", (long)kMaxK);
    IXA_REQUIRE(nprobe > 0 && nprobe <= nlist_, kErrInvalidParam, "nprobe must be > 0 and <= nlist");
    const int nsplit = scan_nsplit(n, nprobe, k, nlist_ > 0 ? ntotal_ / nlist_ * nprobe : 0);
    const int64_t hist_bytes = 2 * 1024 * 4, order_bytes = round_up(n * 8, 256),
                  probes_bytes = round_up(n * nprobe * 4, 256), partial_bytes = nsplit > 1 ? n * nsplit * k * 8 : 0;
    const int64_t need = hist_bytes + order_bytes + probes_bytes + partial_bytes;
    IXA_REQUIRE(need <= (int64_t)kNoAllocScratchBytes, kErrInvalidParam,
                "n = %ld queries with nprobe = %d and k = %ld need %ld bytes of scratch; the static scratch of the "
                "no-allocation entry point holds %zu (use ivfpq_search_probes_device, or fewer queries per call)",
                (long)n, nprobe, (long)k, (long)need, kNoAllocScratchBytes);
    std::lock_guard<std::mutex> lock(g_noalloc_mu);
    // resolved on the first call on a device, not when an index is built: a failure here concerns this entry
    // point only
    unsigned char *base = noalloc_scratch_of_current_device();
    ScanScratch ext{};
    ext.hist = reinterpret_cast<int32_t *>(base);
    ext.order = reinterpret_cast<int32_t *>(base + hist_bytes);
    int32_t *probes = reinterpret_cast<int32_t *>(base + hist_bytes + order_bytes);
    ext.partial = reinterpret_cast<unsigned long long *>(base + hist_bytes + order_bytes + probes_bytes);
    // the array keeps what the last call left: the histogram has to start at zero
    hipLaunchKernelGGL(fill_i32_kernel, dim3(8), dim3(256), 0, stream_, ext.hist, 2 * 1024, 0);
    hipLaunchKernelGGL(sanitize_probes_kernel, dim3(blocks_for(n * nprobe)), dim3(256), 0, stream_, probes_dev,
                       n * nprobe, (int32_t)nlist_, probes);
    ScanParams p = scan_params(x_dev, n, probes, nprobe, k, dist_dev, labels_dev, &ext);
    launch_scan(p, n, stream_);
    sync_stream(stream_);
}

// -------------------------------------------------------------------------------------------------
// search (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2351-2411): the whole batch goes through three
// launches on one stream -- no per-8-query batching, no host round trip for the probe lists.
void IvfpqIndex::search(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device)
{
    check_trained();
    IXA_REQUIRE(x && dist && labels, kErrInvalidParam, "x, distances and labels can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    IXA_REQUIRE(k > 0 && k <= kMaxK, kErrInvalidParam, "k must be > 0 and <= %ld", (long)kMaxK);
    // Query paging (AscendIndexImpl::searchPaged, FR/ascend/impl/AscendIndexImpl.cpp:296-346): the workspaces
    // of a search grow with the number of queries -- staged queries and results (host callers), split
    // operands, probe lists, candidate keys -- and stay within the scratch budget (the reference's
    // resourceSize) by serving a very large batch page by page.  Results do not depend on the paging.
    const int64_t ncand = std::min<int64_t>(nlist_, (int64_t)nprobe_ + 16 + nprobe_ / 8);
    const int64_t per_query = (on_device ? 0 : (int64_t)d_ * 4 + k * 12) + (int64_t)3 * dp_ * 2 + ncand * 8 +
                              (int64_t)nprobe_ * 4 + 64;
    const int64_t page = std::max<int64_t>(256, cfg_.scratch_bytes / per_query / 256 * 256);
    if (n <= page) {
        search_page(n, x, k, dist, labels, on_device);
        return;
    }
    SearchStats total{};
    for (int64_t p0 = 0; p0 < n; p0 += page) {
        const int64_t np = std::min(page, n - p0);
        search_page(np, x + p0 * d_, k, dist + p0 * k, labels + p0 * k, on_device);
        const SearchStats &s = stats();   // of this page (a small launch and a wait: nothing beside a page's work)
        total.scanned_codes += s.scanned_codes;
        total.ms_coarse += s.ms_coarse;
        total.ms_scan += s.ms_scan;
        total.ms_total += s.ms_total;
        total.scan_launches += s.scan_launches;
        total.coarse_reruns += s.coarse_reruns;
        total.nsplit = s.nsplit;
        total.scan_waves = s.scan_waves;
        total.shared_pool = s.shared_pool;
        total.ordered = s.ordered;
        total.coarse_plan = s.coarse_plan;
        total.pages += 1;
    }
    stats_ = total;
}

void IvfpqIndex::search_page(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device)
{
    const float *xd = x;
    // A batch in host memory goes through one page-locked staging buffer (queries | distances | labels): a copy to
    // or from pageable memory costs about 45 us each on its own, whatever its size.
    const size_t in_bytes = (size_t)n * d_ * sizeof(float), dist_bytes = (size_t)n * k * sizeof(float),
                 label_bytes = (size_t)n * k * sizeof(int64_t);
    const size_t dist_at = (in_bytes + 255) / 256 * 256, label_at = dist_at + (dist_bytes + 255) / 256 * 256;
    // (larger batches take the same route with the queries going up in two halves)
    const bool staged_io = !on_device && label_at + label_bytes <= kPipelinedIoBytes;
    const bool pipelined_io = staged_io && label_at + label_bytes > kStagedIoBytes;
    unsigned char *io = nullptr;
    if (staged_io) {
        io = static_cast<unsigned char *>(io_stage_.reserve(label_at + label_bytes));
        ws_x_.resize((size_t)n * d_);
        // the queries go up in two halves when there is much of them: the second half is copied into the staging
        // buffer while the first is on its way
        const size_t half = pipelined_io ? (in_bytes / 2 + 4095) / 4096 * 4096 : in_bytes;
        for (size_t off = 0; off < in_bytes; off += half) {
            const size_t bytes = std::min(half, in_bytes - off);
            parallel_copy({{io + off, reinterpret_cast<const unsigned char *>(x) + off, bytes}});
            IXA_HIP(hipMemcpyAsync(reinterpret_cast<unsigned char *>(ws_x_.data()) + off, io + off, bytes,
                                   hipMemcpyHostToDevice, stream_));
        }
        xd = ws_x_.data();
    } else if (!on_device) {
        ws_x_.upload(x, (size_t)n * d_, stream_);
        xd = ws_x_.data();
    }
    float *dd = dist;
    int64_t *ld = labels;
    if (staged_io) {
        // The kernels that finish a query write its distances and labels straight into the page-locked staging buffer,
        // which the GPU addresses over PCIe: the results travel while other queries are still being scanned, and no
        // copy engine has to be waited for once the last kernel is done.  (Nothing reads the results back.)
        void *mapped = nullptr;
        IXA_HIP(hipHostGetDevicePointer(&mapped, io, 0));
        dd = reinterpret_cast<float *>(static_cast<unsigned char *>(mapped) + dist_at);
        ld = reinterpret_cast<int64_t *>(static_cast<unsigned char *>(mapped) + label_at);
    } else if (!on_device) {
        ws_dist_.resize((size_t)n * k);
        ws_labels_.resize((size_t)n * k);
        dd = ws_dist_.data();
        ld = ws_labels_.data();
    }
    ws_probes_.resize((size_t)n * nprobe_);
    ws_counter_.resize(1);

    const bool timed = cfg_.stage_timings > 0 || (cfg_.stage_timings < 0 && n >= 256);
    if (timed) {
        IXA_HIP(hipEventRecord(ev_[0], stream_));
    }
    last_coarse_reruns_ = 0;
    coarse_select(xd, n, nprobe_, metric_, ws_probes_.data(), nullptr, true, true);
    if (timed) {
        IXA_HIP(hipEventRecord(ev_[1], stream_));
    }

    ScanParams p = scan_params(xd, n, ws_probes_.data(), nprobe_, k, dd, ld);
    const int nsplit = p.nsplit;
    launch_scan(p, n, stream_);
    // the scan is queued; only now does the host look at the coarse stage's verdict.  Queries that had to
    // be redone exactly (near-tied centroids: rare) have new probe lists, and the scan runs again.
    std::vector<int32_t> redone;
    if (coarse_finish(xd, nprobe_, metric_, ws_probes_.data(), nullptr, &redone) > 0) {
        // only the redone queries are scanned again: their rows are the execution order of a second launch
        ws_redo_.upload(redone.data(), redone.size(), stream_);
        ScanParams again = p;
        again.order = ws_redo_.data();
        again.xcd_chunks = 0;
        launch_scan(again, (int64_t)redone.size(), stream_);
    }
    stats_.coarse_reruns = last_coarse_reruns_;
    stats_.coarse_plan = last_coarse_plan_;
    stats_.ordered = p.order ? (p.xcd_chunks ? 2 : 1) : 0;   // 1 = heaviest first, 2 = by locality
    {
        ScanParams planned = p;
        plan_scan(planned);
        stats_.scan_waves = planned.waves;
        stats_.shared_pool = planned.shared_pool;
    }
    if (timed) {
        IXA_HIP(hipEventRecord(ev_[2], stream_));
    }
    stats_timed_ = timed;

    if (staged_io) {
        sync_stream(stream_);
        parallel_copy({{dist, io + dist_at, dist_bytes}, {labels, io + label_at, label_bytes}});
    } else if (!on_device) {
        ws_dist_.download(dist, (size_t)n * k, stream_);
        ws_labels_.download(labels, (size_t)n * k, stream_);
    } else {
        sync_stream(stream_);
    }
    stats_.scan_launches = nsplit > 1 ? 2 : 1;
    stats_.nsplit = nsplit;
    stats_.pages = 1;
    stats_pending_ = true;   // timings and the scanned-code count are worked out when somebody asks
    stats_rows_ = n;
    stats_nprobe_ = nprobe_;
}

// Statistics of the last search.  The event timings and the number of scanned codes (a kernel over
// the probe lists, which stay in the workspace until the next search) are evaluated here, not in
// search(): they cost a launch and a host synchronisation that the search path does not need.
void IvfpqIndex::last_timings(double *ms_coarse, double *ms_scan)
{
    float ms01 = 0, ms12 = 0;
    if (stats_pending_) {   // the events of the last search have completed: search() synchronises its stream
        if (stats_timed_) {
            IXA_HIP(hipEventElapsedTime(&ms01, ev_[0], ev_[1]));
            IXA_HIP(hipEventElapsedTime(&ms12, ev_[1], ev_[2]));
        }
    } else {
        ms01 = (float)stats_.ms_coarse;
        ms12 = (float)stats_.ms_scan;
    }
    if (ms_coarse) {
        *ms_coarse = ms01;
    }
    if (ms_scan) {
        *ms_scan = ms12;
    }
}

const SearchStats &IvfpqIndex::stats()
{
    if (stats_pending_) {
        ws_counter_.resize(1);
        IXA_HIP(hipMemsetAsync(ws_counter_.data(), 0, 8, stream_));
        launch_count_scanned(ws_probes_.data(), stats_rows_ * stats_nprobe_, list_len_dev_.data(), nlist_, ws_counter_.data(),
                             stream_);
        unsigned long long scanned = 0;
        ws_counter_.download(&scanned, 1, stream_);
        float ms01 = 0, ms12 = 0;
        if (stats_timed_) {
            IXA_HIP(hipEventElapsedTime(&ms01, ev_[0], ev_[1]));
            IXA_HIP(hipEventElapsedTime(&ms12, ev_[1], ev_[2]));
        }
        stats_.scanned_codes = (double)scanned;
        stats_.ms_coarse = ms01;
        stats_.ms_scan = ms12;
        stats_.ms_total = ms01 + ms12;
        stats_pending_ = false;
    }
    return stats_;
}

// -------------------------------------------------------------------------------------------------
// Training.  The reference delegates to faiss::Clustering (CPU mode) or runs device assignment with
// a host centroid update (NPU mode: FR/ascendhost/src/impl/AscendClusteringImpl.cpp:686-762); this
// build does the latter: assignment on the GPU (stage-1 kernels, PQ encode kernel); the coarse centroid
// update also runs on the GPU (float64 sums in sample order, so the result does not depend on the
// hardware's scheduling), the sub-quantizer update on the host in float64.  Sampling follows
// computeTrainTotalSize / sampleTrainData (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:51-112).  Plain Lloyd
// unless cfg.spherical.

void IvfpqIndex::train(int64_t n, const float *x, bool on_device)
{
    flush_stats();
    IXA_REQUIRE(x, kErrInvalidParam, "x can not be nullptr.");
    IXA_REQUIRE(n > 0 && n < kMaxN, kErrInvalidParam, "n must be > 0 and < %ld", (long)kMaxN);
    if (trained_) {
        return;  // same as the reference: training a trained index is a no-op
    }
    IXA_REQUIRE(n >= nlist_ && n >= 256, kErrInvalidParam,
                "need at least max(nlist, 256) = %ld training vectors, got %ld", (long)std::max<int64_t>(nlist_, 256),
                (long)n);
    int64_t ns = std::min<int64_t>({(int64_t)nlist_ * cfg_.train_samples_per_list, n, cfg_.max_train_samples});
    ns = std::max<int64_t>(ns, std::min<int64_t>(n, std::max<int64_t>(nlist_, 256 * 40)));
    std::vector<int64_t> idx((size_t)n);
    std::iota(idx.begin(), idx.end(), 0);
    if (ns < n) {
        std::mt19937_64 gen(cfg_.seed);
        std::shuffle(idx.begin(), idx.end(), gen);
        idx.resize((size_t)ns);
    }
    // the sample lives in device memory from here on: rows of a device-resident training set are gathered on
    // the device and never visit the host; a host training set is sampled on the host and uploaded once
    DeviceBuffer<float> sample_dev((size_t)ns * d_);
    if (on_device) {
        DeviceBuffer<int64_t> idx_dev;
        idx_dev.upload(idx.data(), (size_t)ns, stream_);
        hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for(ns * d_)), dim3(256), 0, stream_, x, idx_dev.data(), ns,
                           d_, sample_dev.data());
        sync_stream(stream_);   // idx_dev is freed on leaving this block
    } else {
        std::vector<float> sample((size_t)ns * d_);
        for (int64_t i = 0; i < ns; i++) {
            std::memcpy(&sample[(size_t)i * d_], x + idx[(size_t)i] * d_, sizeof(float) * (size_t)d_);
        }
        sample_dev.upload(sample.data(), sample.size(), stream_);
        sync_stream(stream_);   // the host copy is freed on leaving this block
    }
    kmeans_coarse(sample_dev.data(), ns);
    kmeans_pq(sample_dev.data(), ns);
    trained_ = true;
}

namespace {

// Re-seeds empty clusters by splitting the most populated one (symmetric perturbation).
void split_empty(std::vector<float> &cent, std::vector<int64_t> &cnt, int64_t k, int dim)
{
    for (int64_t c = 0; c < k; c++) {
        if (cnt[(size_t)c] != 0) {
            continue;
        }
        const int64_t big = std::max_element(cnt.begin(), cnt.begin() + k) - cnt.begin();
        for (int t = 0; t < dim; t++) {
            const float v = cent[(size_t)(big * dim + t)];
            const float eps = (t & 1) ? 1.0f / 1024 : -1.0f / 1024;
            cent[(size_t)(c * dim + t)] = v * (1.0f + eps);
            cent[(size_t)(big * dim + t)] = v * (1.0f - eps);
        }
        cnt[(size_t)c] = cnt[(size_t)big] / 2;
        cnt[(size_t)big] -= cnt[(size_t)c];
    }
}

void normalise_rows(std::vector<float> &cent, int64_t k, int dim)
{
    for (int64_t c = 0; c < k; c++) {
        double nn = 0;
        for (int t = 0; t < dim; t++) {
            nn += (double)cent[(size_t)(c * dim + t)] * cent[(size_t)(c * dim + t)];
        }
        nn = std::sqrt(nn);
        if (nn > 0) {
            for (int t = 0; t < dim; t++) {
                cent[(size_t)(c * dim + t)] = (float)(cent[(size_t)(c * dim + t)] / nn);
            }
        }
    }
}

}  // namespace

void IvfpqIndex::kmeans_coarse(const float *sample_dev, int64_t ns)
{
    std::vector<int64_t> pick((size_t)ns);
    std::iota(pick.begin(), pick.end(), 0);
    std::mt19937_64 gen(cfg_.seed + 1);
    std::shuffle(pick.begin(), pick.end(), gen);
    // The first centroids are sample rows, gathered on the device.  From here on an iteration moves nothing of the
    // sample's size between host and device: assignments, the members of every cluster in sample order, the means
    // (float64 sums in exactly that order, one workgroup per centroid), the re-seeding of empty clusters and the
    // normalisation all stay in device memory (only the nlist norms come to the host, for the largest of them).
    centroids_.resize((size_t)nlist_ * d_);
    {
        DeviceBuffer<int64_t> pick_dev;
        pick_dev.upload(pick.data(), (size_t)nlist_, stream_);
        hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for(nlist_ * d_)), dim3(256), 0, stream_, sample_dev,
                           pick_dev.data(), nlist_, d_, centroids_.data());
        sync_stream(stream_);   // pick_dev is freed on leaving this block
    }
    DeviceBuffer<int32_t> asg((size_t)ns);
    DeviceBuffer<unsigned long long> cnt((size_t)nlist_), cursor((size_t)nlist_);
    DeviceBuffer<int64_t> order((size_t)ns), seg((size_t)nlist_ + 1);
    DeviceBuffer<float> mean((size_t)nlist_ * d_);
    const bool spherical = cfg_.spherical < 0 ? metric_ == kMetricInnerProduct : cfg_.spherical != 0;
    for (int it = 0; it < cfg_.niter; it++) {
        derive_from_centroids();
        coarse_select(sample_dev, ns, 1, kMetricL2, asg.data(), nullptr);
        IXA_HIP(hipMemsetAsync(cnt.data(), 0, cnt.bytes(), stream_));
        hipLaunchKernelGGL(count_members_kernel, dim3(blocks_for(ns)), dim3(256), 0, stream_, asg.data(), ns, cnt.data());
        hipLaunchKernelGGL(segment_starts_kernel, dim3(1), dim3(1024), 0, stream_, cnt.data(), nlist_, seg.data(),
                           cursor.data());
        hipLaunchKernelGGL(place_members_kernel, dim3(blocks_for(ns)), dim3(256), 0, stream_, asg.data(), ns,
                           cursor.data(), order.data());
        hipLaunchKernelGGL(sort_segments_kernel, dim3((unsigned)nlist_), dim3(256), 0, stream_, order.data(), seg.data());
        hipLaunchKernelGGL(segment_mean_kernel, dim3((unsigned)nlist_), dim3(d_ <= 64 ? 64 : (d_ <= 128 ? 128 : 256)), 0,
                           stream_, sample_dev, d_, order.data(), seg.data(), centroids_.data(), mean.data());
        hipLaunchKernelGGL(split_empty_kernel, dim3(1), dim3(1024), 0, stream_, mean.data(), cnt.data(), nlist_, d_);
        if (spherical) {
            hipLaunchKernelGGL(normalise_rows_kernel, dim3(blocks_for(nlist_)), dim3(256), 0, stream_, mean.data(), nlist_,
                               d_);
        }
        IXA_HIP(hipMemcpyAsync(centroids_.data(), mean.data(), mean.bytes(), hipMemcpyDeviceToDevice, stream_));
    }
    derive_from_centroids();
    sync_stream(stream_);
}

void IvfpqIndex::kmeans_pq(const float *sample_dev, int64_t ns)
{
    const int niter = cfg_.pq_niter >= 0 ? cfg_.pq_niter : cfg_.niter;
    // the first codewords of sub-quantizer m are the m-th sub-vectors of 256 sample rows: those rows are gathered
    // on the device (M x 256 rows come to the host, not the sample)
    std::vector<float> cb((size_t)M_ * 256 * dsub_);
    std::mt19937_64 gen(cfg_.seed + 2);
    {
        std::vector<int64_t> rows_of((size_t)M_ * 256);
        for (int m = 0; m < M_; m++) {
            std::vector<int64_t> pick((size_t)ns);
            std::iota(pick.begin(), pick.end(), 0);
            std::shuffle(pick.begin(), pick.end(), gen);
            for (int k = 0; k < 256; k++) {
                rows_of[(size_t)m * 256 + k] = pick[(size_t)(k % ns)];
            }
        }
        DeviceBuffer<int64_t> rows_dev;
        DeviceBuffer<float> picked((size_t)M_ * 256 * d_);
        std::vector<float> h_picked((size_t)M_ * 256 * d_);
        rows_dev.upload(rows_of.data(), rows_of.size(), stream_);
        hipLaunchKernelGGL(gather_rows_kernel, dim3(blocks_for((int64_t)M_ * 256 * d_)), dim3(256), 0, stream_,
                           sample_dev, rows_dev.data(), (int64_t)M_ * 256, d_, picked.data());
        picked.download(h_picked.data(), h_picked.size(), stream_);
        for (int m = 0; m < M_; m++) {
            for (int k = 0; k < 256; k++) {
                std::memcpy(&cb[((size_t)m * 256 + k) * dsub_], &h_picked[((size_t)m * 256 + k) * d_ + m * dsub_],
                            sizeof(float) * (size_t)dsub_);
            }
        }
    }
    struct {
        const float *p;
        const float *data() const { return p; }
    } xs{sample_dev};
    std::vector<float> sample;   // host copy of the sample: only the host update of long sub-vectors needs it
    DeviceBuffer<uint8_t> codes((size_t)ns * M_);
    std::vector<uint8_t> h_codes((size_t)ns * M_);
    std::vector<double> acc((size_t)M_ * 256 * dsub_);
    std::vector<int64_t> cnt((size_t)M_ * 256);
    DeviceBuffer<double> acc_dev(acc.size());
    DeviceBuffer<long long> cnt_dev(cnt.size());
    static_assert(sizeof(long long) == sizeof(int64_t), "count buffers are copied as they are");
    for (int it = 0; it < niter; it++) {
        upload_trained(nullptr, cb.data());
        launch_pq_encode(xs.data(), ns, d_, M_, codebook_.data(), codes.data(), stream_);
        // sums per codeword in float64, in sample order: on the device for the usual sub-vector
        // lengths, else by the host loop the kernel restates (same order, same results)
        if (launch_pq_update(xs.data(), codes.data(), ns, d_, M_, dsub_, acc_dev.data(), cnt_dev.data(), stream_)) {
            acc_dev.download(acc.data(), acc.size(), stream_);
            cnt_dev.download(reinterpret_cast<long long *>(cnt.data()), cnt.size(), stream_);
        } else {
            if (sample.empty()) {
                sample.resize((size_t)ns * d_);
                IXA_HIP(hipMemcpyAsync(sample.data(), sample_dev, sample.size() * sizeof(float), hipMemcpyDeviceToHost,
                                       stream_));
                sync_stream(stream_);
            }
            codes.download(h_codes.data(), h_codes.size(), stream_);
            std::fill(acc.begin(), acc.end(), 0.0);
            std::fill(cnt.begin(), cnt.end(), 0);
            for (int64_t i = 0; i < ns; i++) {
                for (int m = 0; m < M_; m++) {
                    const size_t slot = (size_t)m * 256 + h_codes[(size_t)i * M_ + m];
                    cnt[slot]++;
                    for (int t = 0; t < dsub_; t++) {
                        acc[slot * dsub_ + t] += sample[(size_t)i * d_ + m * dsub_ + t];
                    }
                }
            }
        }
        for (int m = 0; m < M_; m++) {
            std::vector<float> sub(cb.begin() + (size_t)m * 256 * dsub_, cb.begin() + (size_t)(m + 1) * 256 * dsub_);
            std::vector<int64_t> sc(cnt.begin() + (size_t)m * 256, cnt.begin() + (size_t)(m + 1) * 256);
            for (int k = 0; k < 256; k++) {
                if (sc[(size_t)k] > 0) {
                    for (int t = 0; t < dsub_; t++) {
                        sub[(size_t)k * dsub_ + t] =
                            (float)(acc[((size_t)m * 256 + k) * dsub_ + t] / (double)sc[(size_t)k]);
                    }
                }
            }
            split_empty(sub, sc, 256, dsub_);
            // cfg_.spherical (the coarse quantizer's flag) is not applied here; the reference's HOST training
            // normalises the sub-quantizers as well (AscendIndexIVFPQImpl.cpp:1064-1067), its device training does
            // not: pq_spherical asks for the former
            if (cfg_.pq_spherical) {
                normalise_rows(sub, 256, dsub_);
            }
            std::copy(sub.begin(), sub.end(), cb.begin() + (size_t)m * 256 * dsub_);
        }
    }
    upload_trained(nullptr, cb.data());
}

}  // namespace ixa
