// Stage operators: the reference's search path is five named device operators driven by
// AscendOperator::exec (FR/ascenddaemon/impl/IndexIVFPQ.cpp:1600-1804, 2104-2160).  The index-level
// entry points fuse them; the launchers below expose three of them one by one -- plain device
// buffers in, plain device buffers out, no allocation, asynchronous on the caller's stream -- for a
// host layer that keeps the reference's own staging, and so that each stage's arithmetic can be
// checked on its own.  All three use the canonical scalar arithmetic (left to right, no FMA).
#include "coarse.h"
#include "ops.h"
#include "topk.h"

namespace ixa {

namespace {

// DistanceFlatL2MinsAtFP32 (FR/ops/ascendc/op_kernel/distance_flat_l2_mins_at_fp32.cpp:191-236): one
// wavefront per (query, burst of 64 codes); lane = code.
//   dist[q][j] = ((|q|^2 + sqr[j]) - g) - g,  g = dot(q, c_j) left to right
//   mins[q][2 b], mins[q][2 b + 1] = smallest distance of burst b and (as the bit pattern of a uint32)
//   its position inside the burst, the first one on ties
__global__ __launch_bounds__(256) void op_distance_l2_mins_kernel(const float *__restrict__ Q, int64_t nq,
                                                                  const float *__restrict__ C, int64_t n, int d,
                                                                  const float *__restrict__ sqr,
                                                                  float *__restrict__ dist, float *__restrict__ mins)
{
    const int lane = threadIdx.x & 63;
    const int64_t bursts = (n + 63) / 64;
    const int64_t burst = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t row = blockIdx.y;
    if (burst >= bursts) {
        return;
    }
    const int64_t col = burst * 64 + lane;
    const float *q = Q + row * d;
    const bool ok = col < n;
    const float *c = C + (ok ? col : n - 1) * d;
    float g = 0.f, qn = 0.f;
    for (int t = 0; t < d; t++) {
        const float qv = q[t];
        g = __fadd_rn(g, __fmul_rn(qv, c[t]));
        qn = __fadd_rn(qn, __fmul_rn(qv, qv));
    }
    float v = __fadd_rn(qn, sqr[ok ? col : n - 1]);
    v = __fsub_rn(v, g);
    v = __fsub_rn(v, g);
    if (ok) {
        dist[row * n + col] = v;
    }
    if (mins) {
        // (value, lane) minimum over the wavefront; lanes past the end never win
        float best = ok ? v : __builtin_inff();
        int where = ok ? lane : 64;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off);
            const int ow = __shfl_xor(where, off);
            if (ob < best || (ob == best && ow < where)) {
                best = ob;
                where = ow;
            }
        }
        if (lane == 0) {
            mins[row * bursts * 2 + burst * 2] = best;
            mins[row * bursts * 2 + burst * 2 + 1] = __uint_as_float((uint32_t)where);
        }
    }
}

// AscendcIvfpqSubspaceDistance (FR/ops/ascendc/op_kernel/ascendc_ivfpq_subspace_distance.cpp:419-463):
//   L2: lut[q][m][k] = (|cb_mk|^2 + |q_m|^2) + (-2 dot(q_m, cb_mk));  inner product: dot(q_m, cb_mk)
__global__ __launch_bounds__(256) void op_subspace_distance_kernel(const float *__restrict__ Q, int64_t nq, int d,
                                                                   const float *__restrict__ codebook, int M, int dsub,
                                                                   int metric, float *__restrict__ lut)
{
    const int kk = threadIdx.x;
    const int m = blockIdx.x;
    const int64_t row = blockIdx.y;
    const float *qm = Q + row * d + m * dsub;
    const float *cw = codebook + ((int64_t)m * 256 + kk) * dsub;
    float ip = 0.f, qn = 0.f, cn = 0.f;
    for (int t = 0; t < dsub; t++) {
        const float qv = qm[t], cv = cw[t];
        ip = __fadd_rn(ip, __fmul_rn(qv, cv));
        qn = __fadd_rn(qn, __fmul_rn(qv, qv));
        cn = __fadd_rn(cn, __fmul_rn(cv, cv));
    }
    const float v = metric == kMetricL2 ? __fadd_rn(__fadd_rn(cn, qn), __fmul_rn(ip, -2.0f)) : ip;
    lut[(row * M + m) * 256 + kk] = v;
}

// keys (in the label buffer) -> distances and labels, in place: every thread reads its key before it
// writes the label over it
__global__ __launch_bounds__(256) void op_topk_finish_kernel(int64_t *__restrict__ labels, float *__restrict__ dist,
                                                             int64_t n)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n) {
        return;
    }
    const key_t kk = reinterpret_cast<const key_t *>(labels)[e];
    const bool ok = kk != kEmptyKey;
    dist[e] = ok ? key_score(kk) : 3.402823466e+38f;
    labels[e] = ok ? (int64_t)key_index(kk) : -1;
}

// AscendcIvfpqSearchDistanceL2 (FR/ascenddaemon/impl/IndexIVFPQ.cpp:1706-1755, kernel
// FR/ops/ascendc/op_kernel/ascendc_ivfpq_search_distance_topk.h:39-93, 556-810) with the reference's operands: the
// per-query LUT that AscendcIvfpqSubspaceDistance wrote, one code base pointer plus per-(query, block) byte
// offsets and valid lengths, one label base pointer plus per-(query, block) element offsets.  One workgroup of
// eight wavefronts per query: LUT into LDS, the blocks form one sequence of 64-code groups dealt to the
// wavefronts, dist = sum over m of lut[m][code[m]] in m order (the reference's scalar order), private candidate
// pools merged at the end.  A candidate's key carries (block << 18 | position), so blocks hold at most 262144
// codes -- the reference's block size (FR/common/utils/CommonUtils.h:57-85).
struct OpScanParams {
    const float *lut;
    const uint8_t *code_base;
    const int64_t *code_offset, *code_size;
    const int64_t *label_base;
    const int64_t *label_offset;
    int nblk, M, k, cap, metric;
    float *out_val;
    int64_t *out_lab;
};

constexpr int kOpScanWaves = 8;
constexpr int kOpScanBlockBits = 18;

__global__ __launch_bounds__(kOpScanWaves * 64) void op_ivfpq_scan_topk_kernel(OpScanParams p)
{
    constexpr int W = kOpScanWaves, NT = W * 64;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float *lut = reinterpret_cast<float *>(smem_raw);
    key_t *pools = reinterpret_cast<key_t *>(smem_raw + (size_t)p.M * 1024);
    float *share = reinterpret_cast<float *>(pools + (size_t)W * p.cap);
    int *counts = reinterpret_cast<int *>(share + W);
    int *t_len = counts + W;
    int *t_gend = t_len + p.nblk;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t q = blockIdx.x;
    const bool ip = p.metric == kMetricInnerProduct;
    for (int i = tid; i < p.M * 256; i += NT) {
        const float v = p.lut[q * p.M * 256 + i];
        lut[i] = ip ? -v : v;   // minimise the negated inner product
    }
    if (tid < W) {
        share[tid] = __builtin_inff();
    }
    for (int i = tid; i < p.nblk; i += NT) {
        const int64_t len = p.code_size[q * p.nblk + i];
        t_len[i] = (int)(len < 0 ? 0 : (len > (1 << kOpScanBlockBits) ? (1 << kOpScanBlockBits) : len));
    }
    __syncthreads();
    if (wave == 0) {
        int carry = 0;
        for (int base = 0; base < p.nblk; base += 64) {
            const int i = base + lane;
            int g = i < p.nblk ? (t_len[i] + 63) >> 6 : 0;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(g, o);
                if (lane >= o) {
                    g += up;
                }
            }
            if (i < p.nblk) {
                t_gend[i] = carry + g;
            }
            carry += __shfl(g, 63);
        }
    }
    __syncthreads();
    WavePool<float> pool;
    pool.init(pools + wave * p.cap, p.cap, p.k);
    const int share_rank = (p.k + W - 1) / W;
    auto adopt_shared = [&]() {
        float b = share[0];
#pragma unroll
        for (int i = 1; i < W; i++) {
            b = fmaxf(b, share[i]);
        }
        b = wave_uniform(b);
        pool.bound = b < pool.bound ? b : pool.bound;
    };
    const int total = __builtin_amdgcn_readfirstlane(t_gend[p.nblk - 1]);
    int li = 0, gstart = 0;
    int gend = __builtin_amdgcn_readfirstlane(t_gend[0]);
    int step = 0;
    for (int G = wave; G < total; G += W, step++) {
        while (G >= gend) {
            gstart = gend;
            li++;
            gend = __builtin_amdgcn_readfirstlane(t_gend[li]);
        }
        const int pos = ((G - gstart) << 6) + lane;
        const bool valid = pos < __builtin_amdgcn_readfirstlane(t_len[li]);
        float s = 0.f;
        if (valid) {
            const uint8_t *cp = p.code_base + p.code_offset[q * p.nblk + li] + (int64_t)pos * p.M;
            if ((p.M & 3) == 0 && (reinterpret_cast<uintptr_t>(cp) & 3) == 0) {
                for (int m = 0; m < p.M; m += 4) {
                    const uint32_t w = *reinterpret_cast<const uint32_t *>(cp + m);
                    s = __fadd_rn(s, lut[m * 256 + (w & 0xffu)]);
                    s = __fadd_rn(s, lut[(m + 1) * 256 + ((w >> 8) & 0xffu)]);
                    s = __fadd_rn(s, lut[(m + 2) * 256 + ((w >> 16) & 0xffu)]);
                    s = __fadd_rn(s, lut[(m + 3) * 256 + (w >> 24)]);
                }
            } else {
                for (int m = 0; m < p.M; m++) {
                    s = __fadd_rn(s, lut[m * 256 + cp[m]]);
                }
            }
        }
        const bool compacted = pool.push(valid && s <= pool.bound, s, ((uint32_t)li << kOpScanBlockBits) | (uint32_t)pos,
                                         lane, &share[wave], share_rank);
        if (compacted || (step & 15) == 0) {
            adopt_shared();
        }
    }
    __syncthreads();   // every wave has published its last value; the LUT is no longer needed
    adopt_shared();
    pool.finish(lane);
    if (lane == 0) {
        counts[wave] = pool.count;
    }
    const int total_keys = block_merge_pools<W>(pools, p.cap, counts, nullptr, 0, tid);
    for (int i = tid; i < p.k; i += NT) {
        const key_t kk = i < total_keys ? pools[i] : kEmptyKey;
        const bool ok = kk != kEmptyKey;
        const float v = key_score(kk);
        float val = ip ? -3.402823466e+38f : 3.402823466e+38f;
        int64_t lab = -1;
        if (ok) {
            const uint32_t idx = key_index(kk);
            const int blk = (int)(idx >> kOpScanBlockBits);
            lab = p.label_base[p.label_offset[q * p.nblk + blk] + (int64_t)(idx & ((1u << kOpScanBlockBits) - 1u))];
            val = ip ? -v : v;
        }
        p.out_val[q * p.k + i] = val;
        p.out_lab[q * p.k + i] = lab;
    }
}

// TopkIvfpqL3 (FR/ops/cpukernel/impl/topk_ivfpq_l3_cpu_kernel.cpp:176-250): merges the best-first lists of T
// tiles per query into the k best.  Entries with label -1 are padding.  One workgroup per query; the union
// (T x K keys) is sorted in LDS.
__global__ __launch_bounds__(256) void op_topk_ivfpq_l3_kernel(const int64_t *__restrict__ in_lab,
                                                               const float *__restrict__ in_val, int T, int64_t batch,
                                                               int K, int k, int asc, int n2,
                                                               float *__restrict__ out_val, int64_t *__restrict__ out_lab)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    key_t *keys = reinterpret_cast<key_t *>(smem_raw);
    const int tid = threadIdx.x;
    const int64_t q = blockIdx.x;
    const int total = T * K;
    for (int e = tid; e < n2; e += 256) {
        key_t kk = kEmptyKey;
        if (e < total) {
            const int t = e / K, pos = e - t * K;
            const int64_t at = ((int64_t)t * batch + q) * K + pos;
            if (in_lab[at] != -1) {
                const float v = in_val[at];
                kk = make_key(asc ? v : -v, (uint32_t)e);
            }
        }
        keys[e] = kk;
    }
    block_bitonic_sort(keys, n2, tid, 256);
    for (int i = tid; i < k; i += 256) {
        const key_t kk = keys[i];
        float val = asc ? 3.402823466e+38f : -3.402823466e+38f;
        int64_t lab = -1;
        if (kk != kEmptyKey) {
            const int e = (int)key_index(kk);
            const int t = e / K, pos = e - t * K;
            const int64_t at = ((int64_t)t * batch + q) * K + pos;
            val = in_val[at];
            lab = in_lab[at];
        }
        out_val[q * k + i] = val;
        out_lab[q * k + i] = lab;
    }
}

}  // namespace

void op_distance_flat_l2_mins_fp32(const float *queries, int64_t batch, const float *codes, int64_t n, int d,
                                   const float *codes_sqr_sum, float *dist, float *mins, hipStream_t s)
{
    IXA_REQUIRE(queries && codes && codes_sqr_sum && dist, kErrInvalidParam, "operator buffers can not be nullptr.");
    IXA_REQUIRE(batch >= 0 && batch <= 65535 && n >= 1 && d >= 1, kErrInvalidParam,
                "DistanceFlatL2MinsAtFP32: batch %ld (<= 65535), codes %ld, dims %d", (long)batch, (long)n, d);
    if (batch == 0) {
        return;
    }
    const int64_t bursts = (n + 63) / 64;
    hipLaunchKernelGGL(op_distance_l2_mins_kernel, dim3((unsigned)((bursts + 3) / 4), (unsigned)batch), dim3(256), 0, s,
                       queries, batch, codes, n, d, codes_sqr_sum, dist, mins);
    IXA_HIP(hipGetLastError());
}

void op_ivfpq_subspace_distance(const float *queries, int64_t batch, int d, const float *codebook, int M, int metric,
                                float *lut, hipStream_t s)
{
    IXA_REQUIRE(queries && codebook && lut, kErrInvalidParam, "operator buffers can not be nullptr.");
    IXA_REQUIRE(batch >= 0 && batch <= 65535 && M >= 1 && d >= M && d % M == 0, kErrInvalidParam,
                "AscendcIvfpqSubspaceDistance: batch %ld (<= 65535), dims %d, msubs %d", (long)batch, d, M);
    IXA_REQUIRE(metric == kMetricL2 || metric == kMetricInnerProduct, kErrInvalidParam, "Unsupported metric type");
    if (batch == 0) {
        return;
    }
    hipLaunchKernelGGL(op_subspace_distance_kernel, dim3((unsigned)M, (unsigned)batch), dim3(256), 0, s, queries, batch,
                       d, codebook, M, d / M, metric, lut);
    IXA_HIP(hipGetLastError());
}

void op_ivfpq_search_distance_topk(const float *lut, int64_t batch, int M, const uint8_t *code_base,
                                   const int64_t *code_offset, const int64_t *code_size, int nblk, int k,
                                   const int64_t *label_base, const int64_t *label_offset, int metric, float *out_val,
                                   int64_t *out_lab, hipStream_t s)
{
    IXA_REQUIRE(lut && code_base && code_offset && code_size && label_base && label_offset && out_val && out_lab,
                kErrInvalidParam, "operator buffers can not be nullptr.");
    IXA_REQUIRE(batch >= 0 && batch <= 65535 && M >= 1 && M <= 128 && nblk >= 1 && nblk <= 2048 && k >= 1 && k <= 384,
                kErrInvalidParam, "AscendcIvfpqSearchDistanceL2: batch %ld (<= 65535), msubs %d (<= 128), blocks %d "
                "(<= 2048), k %d (<= 384)", (long)batch, M, nblk, k);
    IXA_REQUIRE(metric == kMetricL2 || metric == kMetricInnerProduct, kErrInvalidParam, "Unsupported metric type");
    if (batch == 0) {
        return;
    }
    OpScanParams p{lut, code_base, code_offset, code_size, label_base, label_offset, nblk, M, k, 0, metric, out_val, out_lab};
    p.cap = pow2_ceil(k + 128);
    const size_t smem = (size_t)M * 1024 + (size_t)kOpScanWaves * p.cap * sizeof(key_t) + (size_t)kOpScanWaves * 8 +
                        (size_t)nblk * 8;
    IXA_REQUIRE(smem <= 160 * 1024, kErrInvalidParam,
                "AscendcIvfpqSearchDistanceL2: %zu bytes of LDS needed (msubs %d, k %d, %d blocks); the limit is 163840", smem,
                M, k, nblk);
    require_dynamic_lds(reinterpret_cast<const void *>(op_ivfpq_scan_topk_kernel), smem);
    hipLaunchKernelGGL(op_ivfpq_scan_topk_kernel, dim3((unsigned)batch), dim3(kOpScanWaves * 64), smem, s, p);
    IXA_HIP(hipGetLastError());
}

void op_topk_ivfpq_l3(const int64_t *in_labels, const float *in_values, int T, int64_t batch, int K, int k, int asc,
                      float *out_values, int64_t *out_labels, hipStream_t s)
{
    IXA_REQUIRE(in_labels && in_values && out_values && out_labels, kErrInvalidParam, "operator buffers can not be nullptr.");
    IXA_REQUIRE(T >= 1 && K >= 1 && k >= 1 && k <= K && (int64_t)T * K <= 16384 && batch >= 0 && batch <= 65535,
                kErrInvalidParam, "TopkIvfpqL3: %d lists of %d per query (<= 16384 in all), k %d (<= %d), batch %ld", T, K, k,
                K, (long)batch);
    if (batch == 0) {
        return;
    }
    const int n2 = pow2_ceil(T * K);
    const size_t smem = (size_t)n2 * sizeof(key_t);
    require_dynamic_lds(reinterpret_cast<const void *>(op_topk_ivfpq_l3_kernel), smem);
    hipLaunchKernelGGL(op_topk_ivfpq_l3_kernel, dim3((unsigned)batch), dim3(256), smem, s, in_labels, in_values, T, batch,
                       K, k, asc ? 1 : 0, n2, out_values, out_labels);
    IXA_HIP(hipGetLastError());
}

void op_topk_flat_fp32(const float *dists, int64_t batch, int64_t n, int64_t ld, int k, float *out_dist,
                       int64_t *out_label, hipStream_t s)
{
    IXA_REQUIRE(dists && out_dist && out_label, kErrInvalidParam, "operator buffers can not be nullptr.");
    IXA_REQUIRE(batch >= 0 && n >= 1 && ld >= n && k >= 1 && k <= 2048, kErrInvalidParam,
                "TopkFlatFp32: batch %ld, n %ld, ld %ld, k %d (<= 2048)", (long)batch, (long)n, (long)ld, k);
    if (batch == 0) {
        return;
    }
    // the label buffer holds the 64-bit keys until the last kernel splits them
    launch_select_rows(dists, batch, ld, n, k, nullptr, 0, reinterpret_cast<unsigned long long *>(out_label), s, true);
    hipLaunchKernelGGL(op_topk_finish_kernel, dim3((unsigned)((batch * k + 255) / 256)), dim3(256), 0, s, out_label,
                       out_dist, batch * k);
    IXA_HIP(hipGetLastError());
}

}  // namespace ixa
