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
