// Stage 1 of IVFPQ search and the brute-force Flat fp32 path: query x centroid scores on the
// fp32 matrix cores, per-row selection of the best candidates, and an exact re-evaluation of the
// selected candidates in the canonical scalar arithmetic.
//
// Replaces, for one GPU, the reference's L1 level (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2104-2164):
//   op DistanceFlatL2MinsAtFP32 (FR/ops/ascendc/op_kernel/distance_flat_l2_mins_at_fp32.cpp:191-210)
//   op TopkFlatFp32             (FR/ops/cpukernel/impl/topk_flat_fp32_cpu_kernel.cpp:223-384)
//
// "score" everywhere is the value to minimise: the expanded-form L2 distance
// (|q|^2 + |c|^2) - 2 q.c, or the negated inner product.
#include "coarse.h"

#include "topk.h"

namespace ixa {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// ------------------------------------------------------------------------------------------------
// |x_i|^2 accumulated left to right in fp32 (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1114-1126).
// One lane per row: the order of additions is part of the contract, so a row is never split.
__global__ __launch_bounds__(256) void sqnorm_rows_kernel(const float *__restrict__ x, int64_t n, int d,
                                                          float *__restrict__ out)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const float *row = x + i * d;
    float s = 0.0f;
    for (int j = 0; j < d; j++) {
        float v = row[j];
        s = __fadd_rn(s, __fmul_rn(v, v));
    }
    out[i] = s;
}

// The same sums with coalesced loads.  A wavefront serves 16 rows: its 64 lanes fetch 64 columns of
// them at a time (four 128-bit loads per lane, 256 contiguous bytes per row), transpose the chunk
// through LDS, and lanes 0..15 each add their own row's 64 squares in column order; the next chunk's
// loads are in flight meanwhile.  The order of additions per row is unchanged.
__device__ __forceinline__ void sqnorm_rows_tiled_block(const float *__restrict__ x, int64_t n, int d,
                                                        float *__restrict__ out, int64_t block)
{
    __shared__ float tile[4][16][65];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row0 = (block * 4 + wave) * 16;
    if (row0 >= n) {
        return;
    }
    const int cg = lane & 15, rsub = lane >> 4;   // column group of 4, row within a group of 4 rows
    auto fetch = [&](int c0, float4 (&v)[4]) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int64_t r = row0 + rsub + 4 * t;
            const int c = c0 + 4 * cg;
            v[t] = (r < n && c < d) ? *reinterpret_cast<const float4 *>(x + r * d + c) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    float4 cur[4], nxt[4];
    fetch(0, cur);
    float s = 0.0f;
    for (int c0 = 0; c0 < d; c0 += 64) {
        if (c0 + 64 < d) {
            fetch(c0 + 64, nxt);
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            float *p = &tile[wave][rsub + 4 * t][4 * cg];
            p[0] = cur[t].x;
            p[1] = cur[t].y;
            p[2] = cur[t].z;
            p[3] = cur[t].w;
        }
        wave_lds_fence();
        if (lane < 16) {
            const int cols = d - c0 < 64 ? d - c0 : 64;
            for (int j = 0; j < cols; j++) {
                const float v = tile[wave][lane][j];
                s = __fadd_rn(s, __fmul_rn(v, v));
            }
        }
        wave_lds_fence();
#pragma unroll
        for (int t = 0; t < 4; t++) {
            cur[t] = nxt[t];
        }
    }
    if (lane < 16 && row0 + lane < n) {
        out[row0 + lane] = s;
    }
}

__global__ __launch_bounds__(256) void sqnorm_rows_tiled_kernel(const float *__restrict__ x, int64_t n, int d,
                                                                float *__restrict__ out)
{
    sqnorm_rows_tiled_block(x, n, d, out, blockIdx.x);
}

void launch_sqnorm_rows(const float *x, int64_t n, int d, float *out, hipStream_t s)
{
    if (n == 0) {
        return;
    }
    if (d % 4 == 0 && d >= 32 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        hipLaunchKernelGGL(sqnorm_rows_tiled_kernel, dim3((unsigned)((n + 63) / 64)), dim3(256), 0, s, x, n, d, out);
    } else {
        hipLaunchKernelGGL(sqnorm_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, n, d, out);
    }
}

// ---- bf16 x 3 split --------------------------------------------------------------------------------
// x = hi + lo + rest with hi = bf16(x), lo = bf16(x - hi) (both round-to-nearest-even), so
// |lo| <= 2^-9 |x| and |rest| <= 2^-18 |x|.  A dot product over the concatenated rows
// [hi | hi | lo] . [hi | lo | hi]  = hi.hi + hi.lo + lo.hi  misses lo.lo + rest.y + x.rest, at most
// 3 * 2^-18 * sum |x_i y_i|, at three bf16 MFMAs (16x the fp32 matrix rate each) per fp32 product.
// Rows are zero-padded to dp (a multiple of 32) per segment.
__device__ __forceinline__ uint16_t bf16_rne(float v)
{
    uint32_t u = __float_as_uint(v);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ void split_bf16x3_block(const float *__restrict__ x, int64_t n, int d, int dp, int base_side,
                                                   uint16_t *__restrict__ out, int64_t block)
{
    const int64_t e = block * 256 + threadIdx.x;
    if (e >= n * dp) {
        return;
    }
    const int64_t row = e / dp;
    const int j = (int)(e % dp);
    const float v = j < d ? x[row * d + j] : 0.f;
    const uint16_t hi = bf16_rne(v);
    const float hif = __uint_as_float((uint32_t)hi << 16);
    const uint16_t lo = bf16_rne(v - hif);
    uint16_t *o = out + row * 3 * dp + j;
    o[0] = hi;
    o[dp] = base_side ? lo : hi;
    o[2 * dp] = base_side ? hi : lo;
}

__global__ __launch_bounds__(256) void split_bf16x3_kernel(const float *__restrict__ x, int64_t n, int d, int dp,
                                                           int base_side, uint16_t *__restrict__ out)
{
    split_bf16x3_block(x, n, d, dp, base_side, out, blockIdx.x);
}

// Both of the above in one launch (the first blocks add up the norms, the others split): what a search does to its
// queries before the coarse stage's first score launch.
__global__ __launch_bounds__(256) void sqnorm_and_split_kernel(const float *__restrict__ x, int64_t n, int d, int dp,
                                                               float *__restrict__ norms, uint16_t *__restrict__ split,
                                                               unsigned norm_blocks)
{
    if (blockIdx.x < norm_blocks) {
        sqnorm_rows_tiled_block(x, n, d, norms, blockIdx.x);
    } else {
        split_bf16x3_block(x, n, d, dp, 0, split, blockIdx.x - norm_blocks);
    }
}

void launch_sqnorm_and_split_bf16x3(const float *x, int64_t n, int d, int dp, float *norms, uint16_t *split, hipStream_t s)
{
    if (n == 0) {
        return;
    }
    if (d % 4 == 0 && d >= 32 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        const unsigned norm_blocks = (unsigned)((n + 63) / 64), split_blocks = (unsigned)((n * dp + 255) / 256);
        hipLaunchKernelGGL(sqnorm_and_split_kernel, dim3(norm_blocks + split_blocks), dim3(256), 0, s, x, n, d, dp, norms,
                           split, norm_blocks);
    } else {
        launch_sqnorm_rows(x, n, d, norms, s);
        launch_split_bf16x3(x, n, d, dp, false, split, s);
    }
}

void launch_split_bf16x3(const float *x, int64_t n, int d, int dp, bool base_side, uint16_t *out, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(split_bf16x3_kernel, dim3((unsigned)((n * dp + 255) / 256)), dim3(256), 0, s, x, n, d, dp,
                           base_side ? 1 : 0, out);
    }
}

// ------------------------------------------------------------------------------------------------
// Score tile kernel.  One workgroup (4 wavefronts) produces a 128 x 128 tile; each wavefront owns
// a 64 x 64 quadrant as 2 x 2 blocks of v_mfma_f32_32x32x2_f32 (16 accumulator VGPRs per block).
// Operand tiles are staged through LDS in K-steps of 16 with a padded row stride of 20 floats,
// which makes the 128-bit operand reads of 16 consecutive rows hit disjoint banks.  The sum over
// k is order-free, so each lane half (lane/32) owns 8 of the 16 k's of a step and feeds them to 8
// consecutive MFMAs.
constexpr int kTile = 128;
constexpr int kKStep = 16;
constexpr int kLdsStride = 20;

template <bool VEC4>
__device__ __forceinline__ float4 load_k4(const float *row, int k, int d)
{
    if (VEC4) {
        if (k < d) {
            return *reinterpret_cast<const float4 *>(row + k);
        }
        return make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float4 v;
    v.x = k + 0 < d ? row[k + 0] : 0.f;
    v.y = k + 1 < d ? row[k + 1] : 0.f;
    v.z = k + 2 < d ? row[k + 2] : 0.f;
    v.w = k + 3 < d ? row[k + 3] : 0.f;
    return v;
}

// Tile order: 8 consecutive workgroups (one per XCD) take 8 different column tiles, and each XCD
// then walks all row tiles of its column tile, so a column tile is fetched from HBM once and
// re-used out of that XCD's L2 while the (smaller) row operand stays L2-resident everywhere.
__device__ __forceinline__ bool xcd_tile(int64_t b, int tiles_m, int tiles_n, int64_t &tile_m, int64_t &tile_n)
{
    const int64_t gs = (int64_t)8 * tiles_m;
    const int64_t g = b / gs, r = b % gs;
    tile_n = g * 8 + (r & 7);
    tile_m = r >> 3;
    return tile_n < tiles_n;
}

template <bool VEC4, bool FILTER>
__global__ __launch_bounds__(256) void score_tile_kernel(const float *__restrict__ Q, int64_t nq,
                                                         const float *__restrict__ C, int64_t nc, int d,
                                                         const float *__restrict__ qn, const float *__restrict__ cn,
                                                         int metric, float *__restrict__ out, int64_t ldo,
                                                         int tiles_m, int tiles_n, ScoreFilter<float> flt)
{
    __shared__ float As[2][kTile * kLdsStride];
    __shared__ float Bs[2][kTile * kLdsStride];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    int64_t tile_m, tile_n;
    if (!xcd_tile(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n)) {
        return;
    }
    const int64_t i0 = tile_m * kTile, j0 = tile_n * kTile;

    // global -> register mapping: a tile step is 128 rows x 4 float4; thread t moves float4 t, t+256
    const int lrow0 = tid >> 2, lrow1 = (tid + 256) >> 2, lkq = (tid & 3) * 4;
    const int64_t qa0 = i0 + lrow0 < nq ? i0 + lrow0 : nq - 1, qa1 = i0 + lrow1 < nq ? i0 + lrow1 : nq - 1;
    const int64_t cb0 = j0 + lrow0 < nc ? j0 + lrow0 : nc - 1, cb1 = j0 + lrow1 < nc ? j0 + lrow1 : nc - 1;
    const float *qrow0 = Q + qa0 * d, *qrow1 = Q + qa1 * d;
    const float *crow0 = C + cb0 * d, *crow1 = C + cb1 * d;

    floatx16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++) {
#pragma unroll
        for (int b = 0; b < 2; b++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[a][b][r] = 0.f;
            }
        }
    }

    const int nk = (d + kKStep - 1) / kKStep;
    float4 ra0 = load_k4<VEC4>(qrow0, lkq, d), ra1 = load_k4<VEC4>(qrow1, lkq, d);
    float4 rb0 = load_k4<VEC4>(crow0, lkq, d), rb1 = load_k4<VEC4>(crow1, lkq, d);
    *reinterpret_cast<float4 *>(&As[0][lrow0 * kLdsStride + lkq]) = ra0;
    *reinterpret_cast<float4 *>(&As[0][lrow1 * kLdsStride + lkq]) = ra1;
    *reinterpret_cast<float4 *>(&Bs[0][lrow0 * kLdsStride + lkq]) = rb0;
    *reinterpret_cast<float4 *>(&Bs[0][lrow1 * kLdsStride + lkq]) = rb1;
    __syncthreads();

    for (int ks = 0; ks < nk; ks++) {
        const int buf = ks & 1;
        if (ks + 1 < nk) {
            const int k = (ks + 1) * kKStep + lkq;
            ra0 = load_k4<VEC4>(qrow0, k, d);
            ra1 = load_k4<VEC4>(qrow1, k, d);
            rb0 = load_k4<VEC4>(crow0, k, d);
            rb1 = load_k4<VEC4>(crow1, k, d);
        }
        float a[2][8], b[2][8];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            const float *pa = &As[buf][(wr * 64 + blk * 32 + l32) * kLdsStride + half * 8];
            const float *pb = &Bs[buf][(wc * 64 + blk * 32 + l32) * kLdsStride + half * 8];
            float4 a0 = *reinterpret_cast<const float4 *>(pa), a1 = *reinterpret_cast<const float4 *>(pa + 4);
            float4 b0 = *reinterpret_cast<const float4 *>(pb), b1 = *reinterpret_cast<const float4 *>(pb + 4);
            a[blk][0] = a0.x; a[blk][1] = a0.y; a[blk][2] = a0.z; a[blk][3] = a0.w;
            a[blk][4] = a1.x; a[blk][5] = a1.y; a[blk][6] = a1.z; a[blk][7] = a1.w;
            b[blk][0] = b0.x; b[blk][1] = b0.y; b[blk][2] = b0.z; b[blk][3] = b0.w;
            b[blk][4] = b1.x; b[blk][5] = b1.y; b[blk][6] = b1.z; b[blk][7] = b1.w;
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
#pragma unroll
            for (int ra = 0; ra < 2; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    acc[ra][rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[ra][t], b[rb][t], acc[ra][rb], 0, 0, 0);
                }
            }
        }
        if (ks + 1 < nk) {
            const int nb = buf ^ 1;
            *reinterpret_cast<float4 *>(&As[nb][lrow0 * kLdsStride + lkq]) = ra0;
            *reinterpret_cast<float4 *>(&As[nb][lrow1 * kLdsStride + lkq]) = ra1;
            *reinterpret_cast<float4 *>(&Bs[nb][lrow0 * kLdsStride + lkq]) = rb0;
            *reinterpret_cast<float4 *>(&Bs[nb][lrow1 * kLdsStride + lkq]) = rb1;
        }
        __syncthreads();
    }

    // epilogue: accumulator register r of lane (half, l32) in block (ra, rb) is
    //   row = 8 * (r / 4) + 4 * half + (r % 4),  col = l32   of that 32 x 32 block.
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
        const int64_t col = j0 + wc * 64 + rb * 32 + l32;
        const float cnv = (metric == kMetricL2 && col < nc) ? cn[col] : 0.f;
#pragma unroll
        for (int ra = 0; ra < 2; ra++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t row = i0 + wr * 64 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (row < nq && col < nc) {
                    float g = acc[ra][rb][r];
                    float v;
                    if (metric == kMetricL2) {
                        v = __fadd_rn(qn[row], cnv);
                        v = __fsub_rn(v, g);
                        v = __fsub_rn(v, g);
                    } else {
                        v = -g;
                    }
                    if (FILTER) {
                        if (v <= flt.tau[row]) {
                            const int pos = atomicAdd(&flt.cnt[row], 1);
                            if (pos < flt.cap) {
                                flt.cand[row * flt.cap + pos] = make_key(v, (uint32_t)(col + flt.col_base));
                            }
                        }
                    } else {
                        out[row * ldo + col] = v;
                    }
                }
            }
        }
    }
}

template <bool FILTER>
static void launch_score_tiles_t(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                                 const float *cn, int metric, float *out, int64_t ldo, ScoreFilter<float> flt,
                                 hipStream_t s)
{
    if (nq == 0 || nc == 0) {
        return;
    }
    if (launch_score_ring_f32(Q, nq, C, nc, d, qn, cn, metric, out, ldo, FILTER, flt, s)) {
        return;
    }
    const int64_t tiles_m = (nq + kTile - 1) / kTile, tiles_n = (nc + kTile - 1) / kTile;
    const int64_t nblocks = (tiles_n + 7) / 8 * 8 * tiles_m;
    IXA_REQUIRE(nblocks < (int64_t)1 << 31 && tiles_m < (1 << 28), kErrInvalidParam, "score tile grid too large");
    const bool vec4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(Q) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    dim3 grid((unsigned)nblocks), block(256);
    if (vec4) {
        hipLaunchKernelGGL((score_tile_kernel<true, FILTER>), grid, block, 0, s, Q, nq, C, nc, d, qn, cn, metric, out,
                           ldo, (int)tiles_m, (int)tiles_n, flt);
    } else {
        hipLaunchKernelGGL((score_tile_kernel<false, FILTER>), grid, block, 0, s, Q, nq, C, nc, d, qn, cn, metric, out,
                           ldo, (int)tiles_m, (int)tiles_n, flt);
    }
}

void launch_score_tiles(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                        const float *cn, int metric, float *out, int64_t ldo, hipStream_t s)
{
    launch_score_tiles_t<false>(Q, nq, C, nc, d, qn, cn, metric, out, ldo, ScoreFilter<float>{}, s);
}

void launch_score_tiles_filtered(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                                 const float *cn, int metric, ScoreFilter<float> flt, hipStream_t s)
{
    launch_score_tiles_t<true>(Q, nq, C, nc, d, qn, cn, metric, nullptr, 0, flt, s);
}

// ------------------------------------------------------------------------------------------------
// Merge of filtered candidates into the running best-k keys of each row (one workgroup per row).
template <typename S>
__global__ __launch_bounds__(256) void merge_candidates_kernel(key_t *__restrict__ running, int k, ScoreFilter<S> flt,
                                                               S *__restrict__ tau, int *__restrict__ overflow,
                                                               S *__restrict__ thr, const S *__restrict__ qn, S max_bound)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    key_t *buf = reinterpret_cast<key_t *>(smem_raw);
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    int n = flt.cnt[row];
    if (n == 0) {
        return;  // nothing was admitted for this row in this chunk
    }
    if (n > flt.cap) {
        if (tid == 0) {
            *overflow = 1;
        }
        n = flt.cap;
    }
    key_t *run = running + row * k;
    const int total = k + n;
    int p2 = 2;
    while (p2 < total) {
        p2 <<= 1;
    }
    for (int i = tid; i < p2; i += 256) {
        buf[i] = i < k ? run[i] : (i < total ? flt.cand[row * flt.cap + (i - k)] : kEmptyKey);
    }
    block_bitonic_sort(buf, p2, tid, 256);
    for (int i = tid; i < k; i += 256) {
        run[i] = buf[i];
    }
    if (tid == 0) {
        flt.cnt[row] = 0;
        if (buf[k - 1] != kEmptyKey) {
            const S t = key_score_as<S>(buf[k - 1]);
            tau[row] = t;
            if (thr) {   // the next filtered launch's threshold (exact integer scores): min(tau, max_bound) - |q|^2
                thr[row] = (t < max_bound ? t : max_bound) - qn[row];
            }
        }
    }
}

template <typename S>
static void launch_merge_candidates_t(key_t *running, int k, ScoreFilter<S> flt, S *tau, int64_t nq, int *overflow,
                                      hipStream_t s, S *thr = nullptr, const S *qn = nullptr, S max_bound = S())
{
    if (nq == 0) {
        return;
    }
    const size_t smem = (size_t)pow2_ceil(k + flt.cap) * sizeof(key_t);
    IXA_REQUIRE(smem <= 160 * 1024, kErrInvalidParam, "candidate merge of %d + %d keys exceeds LDS", k, flt.cap);
    require_dynamic_lds(reinterpret_cast<const void *>(merge_candidates_kernel<S>), smem);
    hipLaunchKernelGGL(merge_candidates_kernel<S>, dim3((unsigned)nq), dim3(256), smem, s, running, k, flt, tau,
                       overflow, thr, qn, max_bound);
}

void launch_merge_candidates(unsigned long long *running, int k, ScoreFilter<float> flt, float *tau, int64_t nq,
                             int *overflow, hipStream_t s)
{
    launch_merge_candidates_t<float>(running, k, flt, tau, nq, overflow, s);
}

void launch_merge_candidates_i32(unsigned long long *running, int k, ScoreFilter<int32_t> flt, int32_t *tau,
                                 int64_t nq, int *overflow, hipStream_t s, int32_t *thr, const int32_t *qn,
                                 int32_t max_bound)
{
    launch_merge_candidates_t<int32_t>(running, k, flt, tau, nq, overflow, s, thr, qn, max_bound);
}

// ------------------------------------------------------------------------------------------------
// Per-row selection of the ksel smallest scores of a materialised score row.  One workgroup per
// row, four wavefront pools, block merge.  Optionally the row's running best keys (from earlier
// column chunks) take part in the merge and provide the initial bound, which turns a sequence of
// calls over column chunks into a streaming top-k.  Output: ksel column indices per row (best
// first, -1 where the row has fewer than ksel columns) and/or the keys themselves.
// Keys the pool region of a streaming selection holds: the pools of the scanning wavefronts plus the
// running keys merged in at the end, rounded up to the power of two the merge sorts.
__host__ __device__ inline int select_region_keys(int active, int cap, int extra)
{
    int n = 2;
    while (n < active * cap + extra) {
        n <<= 1;
    }
    return n;
}

template <typename S, int active = 4>
__device__ __forceinline__ void select_row_streaming(unsigned char *smem_raw, const S *__restrict__ scores, int64_t ld,
                                                     int64_t nc, int ksel, int cap, int32_t *__restrict__ out_idx,
                                                     int64_t col_base, key_t *__restrict__ running, bool fresh)
{
    // `active` of the four wavefronts scan (each with a private pool of `cap` keys), all four merge: a
    // selection too large for four pools in LDS runs on two or one
    key_t *pools = reinterpret_cast<key_t *>(smem_raw);                 // select_region_keys() keys
    const int region = select_region_keys(active, cap, running ? ksel : 0);
    // fresh: `running` only receives the result (its content is unspecified on entry)
    S *share = reinterpret_cast<S *>(pools + region);                   // 4
    int *counts = reinterpret_cast<int *>(share + 4);                   // 4

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const S *row = scores + (int64_t)blockIdx.x * ld;
    key_t *run = running ? running + (int64_t)blockIdx.x * ksel : nullptr;
    S start = ScoreOps<S>::worst();
    if (run && !fresh) {
        const key_t last = run[ksel - 1];
        if (last != kEmptyKey) {
            start = key_score_as<S>(last);
        }
    }
    if (tid < 4) {
        share[tid] = ScoreOps<S>::worst();
    }
    __syncthreads();
    const bool scans = wave < active;
    WavePool<S> pool;
    pool.init(pools + (scans ? wave : 0) * cap, cap, ksel);
    pool.bound = wave_uniform(start);
    const int share_rank = (ksel + active - 1) / active;
    auto adopt_shared = [&]() {
        S b = share[0];
        for (int i = 1; i < active; i++) {
            b = share[i] > b ? share[i] : b;
        }
        b = wave_uniform(b);
        pool.bound = b < pool.bound ? b : pool.bound;
    };
    const bool vec4 = (ld % 4 == 0) && (reinterpret_cast<uintptr_t>(scores) % 16 == 0);
    int iter = 0;
    if (!scans) {
        // no work for this wavefront until the merge
    } else if (vec4) {
        // 128-bit loads: a wavefront covers 256 consecutive columns per step
        for (int64_t base = (int64_t)wave * 256; base < nc; base += active * 256, iter++) {
            const int64_t c = base + lane * 4;
            S v[4];
            if (c + 3 < nc) {
                const uint4 u = *reinterpret_cast<const uint4 *>(row + c);
                v[0] = __builtin_bit_cast(S, u.x);
                v[1] = __builtin_bit_cast(S, u.y);
                v[2] = __builtin_bit_cast(S, u.z);
                v[3] = __builtin_bit_cast(S, u.w);
            } else {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    v[t] = c + t < nc ? row[c + t] : ScoreOps<S>::worst();
                }
            }
            bool pass[4];
            bool any = false;
#pragma unroll
            for (int t = 0; t < 4; t++) {
                pass[t] = c + t < nc && v[t] <= pool.bound;
                any |= pass[t];
            }
            bool compacted = false;
            if (__ballot(any)) {
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    compacted |= pool.push(pass[t], v[t], (uint32_t)(c + t + col_base), lane, &share[wave], share_rank);
                }
            }
            if (compacted || (iter & 3) == 3) {
                adopt_shared();
            }
        }
    } else {
        for (int64_t base = (int64_t)wave * 64; base < nc; base += active * 64, iter++) {
            int64_t c = base + lane;
            S v = c < nc ? row[c] : ScoreOps<S>::worst();
            const bool compacted =
                pool.push(c < nc && v <= pool.bound, v, (uint32_t)(c + col_base), lane, &share[wave], share_rank);
            if (compacted || (iter & 7) == 7) {
                adopt_shared();
            }
        }
    }
    __syncthreads();
    if (scans) {
        adopt_shared();
        pool.finish(lane);
    }
    if (lane == 0) {
        counts[wave] = scans ? pool.count : 0;
    }
    const int total = block_merge_pools<4>(pools, cap, counts, run, (run && !fresh) ? ksel : 0, tid);
    for (int i = tid; i < ksel; i += 256) {
        key_t kk = i < total ? pools[i] : kEmptyKey;
        if (out_idx) {
            out_idx[(int64_t)blockIdx.x * ksel + i] = kk == kEmptyKey ? -1 : (int32_t)key_index(kk);
        }
        if (run) {
            run[i] = kk;
        }
    }
}

template <typename S, int ACTIVE>
__global__ __launch_bounds__(256) void select_rows_kernel(const S *__restrict__ scores, int64_t ld, int64_t nc,
                                                          int ksel, int cap, int32_t *__restrict__ out_idx,
                                                          int64_t col_base, key_t *__restrict__ running, bool fresh)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    select_row_streaming<S, ACTIVE>(smem_raw, scores, ld, nc, ksel, cap, out_idx, col_base, running, fresh);
}

// ------------------------------------------------------------------------------------------------
// The same selection for rows of >= 4096 columns and ksel <= 384, built around registers instead of
// pools.  The workgroup loads a segment of 16384 columns at once (64 values per lane, all loads in
// flight together), and needs a bound B with at least ksel values at or below it before it can
// discard anything.  The first segment gets B from group minima: every lane reduces its values to G
// group minima, every wave finds the ceil(ksel / 4)-th smallest of its 64 G minima (that many values
// of the wave lie at or below it), and B is the largest of the four: with the rank near a third of
// the group count only about 1.3 ksel values of the segment pass.  Passing values are appended to a
// candidate list in LDS (ballot compaction per wave), and after every segment that added something
// the list is reduced to its ksel smallest keys in order, by counting ranks (keys are distinct):
// that list is the running result, and its last score is the next segment's B.  Rows with so many
// equal scores that the list overflows are redone by the streaming selection above; the result is
// the same set of keys in either case: the ksel smallest (score, column) keys of the row and of
// `running`.
#ifndef IXA_SELREG_WAVES
#define IXA_SELREG_WAVES 4
#endif
constexpr int kSelRegSeg = 16384;     // columns per segment: 64 per lane
constexpr int kSelRegStage = 160;     // new candidates per wave and segment
constexpr int kSelRegMaxK = 384;
static_assert(kFoldMaxK == kSelRegMaxK, "the record fold ranks with the register selection's key arrays");
constexpr int kSelRegCap = kSelRegMaxK + 4 * kSelRegStage;   // 1024

// dst[0 .. min(n, keep)) = the smallest keys of src[0 .. n) in ascending order, by counting ranks (the
// keys are distinct).  src[0 .. have) is already ascending: those keys know their rank among
// themselves, the others find theirs among them by bisection, and only the n - have new keys are
// counted against one by one.  n <= 256 E, src is 16-byte aligned with src[n] writable; all 256
// threads call it; barriers inside.
template <int E = 4>
__device__ __forceinline__ void rank_select_256(key_t *src, int have, int n, key_t *dst, int keep, int tid)
{
    const int first = have & ~1;              // new keys are read in aligned pairs from here on
    if (tid == 0 && (n & 1)) {
        src[n] = kEmptyKey;                   // never below a key
    }
    __syncthreads();
    key_t mine[E];
    int rank[E];
    const int owned = (n + 255 - tid) >> 8;   // entries tid, tid + 256, ... below n
#pragma unroll
    for (int e = 0; e < E; e++) {
        const int i = tid + 256 * e;
        mine[e] = i < n ? src[i] : 0;         // 0: its rank is not used
        if (i < have) {
            rank[e] = i - (first < have ? (src[first] < mine[e]) : 0);   // src[first] is counted again below
        } else {
            int lo = 0, hi = have;            // keys of the sorted part below mine
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (src[mid] < mine[e]) {
                    lo = mid + 1;
                } else {
                    hi = mid;
                }
            }
            rank[e] = lo - (first < have && first < lo ? 1 : 0);
        }
    }
    const ulonglong2 *pairs = reinterpret_cast<const ulonglong2 *>(src);
    if (n <= 256) {
        for (int f = first >> 1; f < (n + 1) >> 1; f++) {
            const ulonglong2 pr = pairs[f];   // same address in every lane: one broadcast read
            rank[0] += (pr.x < mine[0]) + (pr.y < mine[0]);
        }
    } else if (n <= 512) {
        for (int f = first >> 1; f < (n + 1) >> 1; f++) {
            const ulonglong2 pr = pairs[f];
            rank[0] += (pr.x < mine[0]) + (pr.y < mine[0]);
            rank[1] += (pr.x < mine[1]) + (pr.y < mine[1]);
        }
    } else if (n <= 1024 || E <= 4) {
        for (int f = first >> 1; f < (n + 1) >> 1; f++) {
            const ulonglong2 pr = pairs[f];
#pragma unroll
            for (int e = 0; e < (E < 4 ? E : 4); e++) {
                rank[e] += (pr.x < mine[e]) + (pr.y < mine[e]);
            }
        }
    } else {
        for (int f = first >> 1; f < (n + 1) >> 1; f++) {
            const ulonglong2 pr = pairs[f];
#pragma unroll
            for (int e = 0; e < E; e++) {
                rank[e] += (pr.x < mine[e]) + (pr.y < mine[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < E; e++) {
        if (e < owned && rank[e] < keep) {
            dst[rank[e]] = mine[e];
        }
    }
    __syncthreads();
}

template <typename S, int G>
__global__ __launch_bounds__(256, IXA_SELREG_WAVES) void select_rows_reg_kernel(
    const S *__restrict__ scores, int64_t ld, int64_t nc, int ksel, int cap, int32_t *__restrict__ out_idx,
    int64_t col_base, key_t *__restrict__ running, bool fresh)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    key_t *cand = reinterpret_cast<key_t *>(smem_raw);            // kSelRegCap + 2
    key_t *best = cand + kSelRegCap + 2;                          // kSelRegMaxK
    key_t *stage = best + kSelRegMaxK;                            // 4 x kSelRegStage
    S *gm = reinterpret_cast<S *>(stage + 4 * kSelRegStage);      // 4 x 64 G group minima
    S *wb = gm + 4 * 64 * G;                                      // 4 wave bounds
    int *ctl = reinterpret_cast<int *>(wb + 4);                   // [0..3] new candidates per wave, [4] overflow
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const S *row = scores + (int64_t)blockIdx.x * ld;
    key_t *run = running ? running + (int64_t)blockIdx.x * ksel : nullptr;

    // the running result so far (sorted, kEmptyKey-padded) opens the candidate list
    int have = 0;   // workgroup-uniform: keys in cand[] before this segment, sorted
    if (run && !fresh) {
        for (int i = tid; i < ksel; i += 256) {
            cand[i] = run[i];
        }
        __syncthreads();
        int lo = 0, hi = ksel;   // valid keys form a prefix
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (cand[mid] != kEmptyKey) {
                lo = mid + 1;
            } else {
                hi = mid;
            }
        }
        have = lo;
    }
    bool bounded = have >= ksel;
    S B = bounded ? key_score_as<S>(cand[ksel - 1]) : ScoreOps<S>::worst();
    if (tid == 0) {
        ctl[4] = 0;
    }
    __syncthreads();

    for (int64_t seg0 = 0; seg0 < nc; seg0 += kSelRegSeg) {
        S v[16][4];
        const S *seg = row + seg0;
        const int lim = (int)(nc - seg0 < kSelRegSeg ? nc - seg0 : kSelRegSeg);   // valid columns of the segment
        if (lim == kSelRegSeg) {
            // whole segment: sixteen 128-bit loads per lane, all in flight together
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const uint4 u = *reinterpret_cast<const uint4 *>(seg + (i * 256 + tid) * 4);
                v[i][0] = __builtin_bit_cast(S, u.x);
                v[i][1] = __builtin_bit_cast(S, u.y);
                v[i][2] = __builtin_bit_cast(S, u.z);
                v[i][3] = __builtin_bit_cast(S, u.w);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int c = (i * 256 + tid) * 4;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    v[i][t] = c + t < lim ? seg[c + t] : ScoreOps<S>::worst();
                }
            }
        }
        if (!bounded) {
            // group j of this lane: its loads i with i % G == j
            S mine[G];
#pragma unroll
            for (int j = 0; j < G; j++) {
                S m = ScoreOps<S>::worst();
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    if ((i & (G - 1)) == j) {
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            m = v[i][t] < m ? v[i][t] : m;
                        }
                    }
                }
                mine[j] = m;
                gm[wave * 64 * G + j * 64 + lane] = m;
            }
            wave_lds_fence();
            // how many of the wave's minima lie at or below each of mine
            int below[G];
#pragma unroll
            for (int j = 0; j < G; j++) {
                below[j] = 0;
            }
            const uint4 *quads = reinterpret_cast<const uint4 *>(gm + wave * 64 * G);
            for (int f = 0; f < 16 * G; f++) {
                const uint4 u = quads[f];   // same address in every lane: one broadcast read
                const S x0 = __builtin_bit_cast(S, u.x), x1 = __builtin_bit_cast(S, u.y);
                const S x2 = __builtin_bit_cast(S, u.z), x3 = __builtin_bit_cast(S, u.w);
#pragma unroll
                for (int j = 0; j < G; j++) {
                    below[j] += (x0 <= mine[j]) + (x1 <= mine[j]) + (x2 <= mine[j]) + (x3 <= mine[j]);
                }
            }
            // the smallest of the wave's minima with at least ceil(ksel / 4) minima at or below it
            const int need = (ksel + 3) >> 2;
            S wbound = ScoreOps<S>::worst();
#pragma unroll
            for (int j = 0; j < G; j++) {
                if (below[j] >= need && mine[j] < wbound) {
                    wbound = mine[j];
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const S o = __shfl_xor(wbound, off);
                wbound = o < wbound ? o : wbound;
            }
            if (lane == 0) {
                wb[wave] = wbound;
            }
            __syncthreads();
            B = wb[0];
#pragma unroll
            for (int w = 1; w < 4; w++) {
                B = wb[w] > B ? wb[w] : B;
            }
        }
        // ballot compaction of the passing values into this wave's staging area
        int added = 0;   // wave-uniform
        {
            const uint32_t first_col = (uint32_t)(seg0 + col_base);
            key_t *mystage = stage + wave * kSelRegStage;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int c = (i * 256 + tid) * 4;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const bool pass = v[i][t] <= B && c + t < lim;
                    const unsigned long long mask = __ballot(pass);
                    if (mask) {
                        const int pos = added + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                               __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                        if (pass && pos < kSelRegStage) {
                            mystage[pos] = make_key(v[i][t], first_col + (uint32_t)(c + t));
                        }
                        added += __builtin_popcountll(mask);
                    }
                }
            }
        }
        if (lane == 0) {
            ctl[wave] = added;
            if (added > kSelRegStage) {
                ctl[4] = 1;
            }
        }
        __syncthreads();
        if (ctl[4]) {
            // too many equal scores for the list: the streaming selection redoes the row
            __syncthreads();
            select_row_streaming<S>(smem_raw, scores, ld, nc, ksel, cap, out_idx, col_base, running, fresh);
            return;
        }
        int before = have, total = 0;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int cw = ctl[w];
            before += w < wave ? cw : 0;
            total += cw;
        }
        if (total > 0) {
            for (int i = lane; i < added; i += 64) {
                cand[before + i] = stage[wave * kSelRegStage + i];
            }
            const int n = have + total;
            rank_select_256(cand, have, n, best, ksel, tid);
            have = n < ksel ? n : ksel;
            for (int i = tid; i < have; i += 256) {
                cand[i] = best[i];
            }
            bounded = have >= ksel;
            if (bounded) {
                B = key_score_as<S>(best[ksel - 1]);
            }
        }
        __syncthreads();
    }
    for (int i = tid; i < ksel; i += 256) {
        const key_t kk = i < have ? cand[i] : kEmptyKey;
        if (out_idx) {
            out_idx[(int64_t)blockIdx.x * ksel + i] = kk == kEmptyKey ? -1 : (int32_t)key_index(kk);
        }
        if (run) {
            run[i] = kk;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Fold of the records a record-mode score launch over the WHOLE base appended (runs of four
// consecutive columns whose smallest score was at or below the row's bound tau) into the row's best-k
// keys, sorted, with the proof that makes a bound of ANY origin safe: every score <= tau of the base is
// in the records, so if they hold at least k scores <= tau, their k smallest keys are the k smallest of
// the whole base.  A row without that proof (or with dropped records) is appended to
// flag[1 + flag[0]++] and its last key is set to kEmptyKey, which is how the later stages recognise a
// list they must not judge.  One workgroup per row; k <= kSelRegMaxK.
constexpr int kFoldCap = 2048;   // scores <= tau the fold ranks at once

// Records of the resident-query launch hold the dot products g of a run, not its scores: the score in the
// arithmetic of the score kernels, (|q|^2 + |c|^2) - g - g, or -g for inner product.
__device__ __forceinline__ void record_scores(float (&v)[4], bool raw, int metric, float qnorm,
                                              const float *__restrict__ cn, uint32_t col)
{
    if (!raw) {
        return;
    }
    if (metric == kMetricL2) {
        const float4 c4 = *reinterpret_cast<const float4 *>(cn + col);   // runs start at multiples of four
        const float c[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            float w = __fadd_rn(qnorm, c[t]);
            w = __fsub_rn(w, v[t]);
            v[t] = __fsub_rn(w, v[t]);
        }
    } else {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            v[t] = -v[t];
        }
    }
}

__global__ __launch_bounds__(256) void fold_records_kernel(key_t *__restrict__ running, int k, ScoreFilter<float> flt,
                                                           int *__restrict__ flag, int64_t row_base, bool raw, int metric,
                                                           const float *__restrict__ qn, const float *__restrict__ cn)
{
    __shared__ __align__(16) key_t cand[kFoldCap + 2];
    __shared__ __align__(16) key_t best[kSelRegMaxK];
    __shared__ int n_keys;
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    int nrec = flt.cnt[row];
    bool lost = false;        // workgroup-uniform: something admitted is not among the keys
    if (nrec > flt.cap) {
        nrec = flt.cap;
        lost = true;
    }
    if (tid == 0) {
        n_keys = 0;
    }
    __syncthreads();
    const float tau = flt.tau[row];
    const unsigned char *records = reinterpret_cast<const unsigned char *>(flt.cand) + (int64_t)row * flt.cap * 32;
    for (int r = tid; r < nrec; r += 256) {
        const float4 sc = *reinterpret_cast<const float4 *>(records + (int64_t)r * 32);
        const uint32_t col = *reinterpret_cast<const uint32_t *>(records + (int64_t)r * 32 + 16);
        float v[4] = {sc.x, sc.y, sc.z, sc.w};
        record_scores(v, raw, metric, raw ? qn[row] : 0.f, cn, col);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            if (v[t] <= tau) {
                const int pos = atomicAdd(&n_keys, 1);
                if (pos < kFoldCap) {
                    cand[pos] = make_key(v[t], col + (uint32_t)t);
                }
            }
        }
    }
    __syncthreads();
    int n = n_keys;
    if (n > kFoldCap) {
        n = kFoldCap;
        lost = true;
    }
    if (n <= 1024) {
        rank_select_256<4>(cand, 0, n, best, k, tid);
    } else {
        rank_select_256<8>(cand, 0, n, best, k, tid);
    }
    // proof: at least k scores at or below the bound the launch admitted by
    const bool proven = !lost && n >= k;
    key_t *run = running + row * k;
    for (int i = tid; i < k; i += 256) {
        key_t kk = i < n ? best[i] : kEmptyKey;
        if (!proven && i == k - 1) {
            kk = kEmptyKey;
        }
        run[i] = kk;
    }
    if (tid == 0) {
        flt.cnt[row] = 0;
        if (!proven) {
            flag[1 + atomicAdd(flag, 1)] = (int)(row_base + row);
        }
    }
}

void launch_fold_records(unsigned long long *running, int k, ScoreFilter<float> flt, int64_t nq, int *flag,
                         int64_t row_base, hipStream_t s, const RawRecords *raw)
{
    if (nq == 0) {
        return;
    }
    IXA_REQUIRE(k >= 1 && k <= kSelRegMaxK && k < kFoldCap, kErrInner, "record fold of %d keys", k);
    hipLaunchKernelGGL(fold_records_kernel, dim3((unsigned)nq), dim3(256), 0, s, running, k, flt, flag, row_base,
                       raw != nullptr, raw ? raw->metric : kMetricL2, raw ? raw->qn : nullptr, raw ? raw->cn : nullptr);
}

// tau[row] = the `rank`-th smallest (1-based) of the row's G group minima gm[row * G .. + G): an upper bound
// of the rank-th smallest score of the columns the groups cover.  One wavefront per row, the minima in
// registers, bisection over the ordered score bits.  G <= 64 E.
template <int E>
__global__ __launch_bounds__(256) void tau_from_minima_kernel(const float *__restrict__ gm, int G, int rank, int64_t n,
                                                              float *__restrict__ tau, RecordTest test)
{
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) {
        return;
    }
    uint32_t u[E];
#pragma unroll
    for (int e = 0; e < E; e++) {
        const int i = e * 64 + lane;
        u[e] = i < G ? ordered_bits(gm[row * G + i]) : 0xffffffffu;
    }
    uint32_t p = 0;   // the largest value with fewer than `rank` minima below it = the rank-th smallest
    for (int bit = 31; bit >= 0; bit--) {
        const uint32_t c = p | (1u << bit);
        int below = 0;
#pragma unroll
        for (int e = 0; e < E; e++) {
            below += __popcll(__ballot(u[e] < c));
        }
        p = below < rank ? c : p;
    }
    if (lane == 0) {
        const float t = unordered_bits(p);
        tau[row] = t;
        if (test.out) {
            test.out[row] = record_test_value(test.qn[row], t, test.cmax, test.metric == kMetricL2);
        }
    }
}

void launch_tau_from_minima(const float *gm, int G, int rank, int64_t nq, float *tau, hipStream_t s, const RecordTest *test)
{
    const RecordTest rt = test ? *test : RecordTest{nullptr, 0.f, 0, nullptr};
    if (nq == 0) {
        return;
    }
    IXA_REQUIRE(G >= 1 && G <= 512 && rank >= 1 && rank <= G, kErrInner, "rank %d of %d group minima", rank, G);
    const dim3 grid((unsigned)((nq + 3) / 4)), block(256);
    if (G <= 64) {
        hipLaunchKernelGGL(tau_from_minima_kernel<1>, grid, block, 0, s, gm, G, rank, nq, tau, rt);
    } else if (G <= 128) {
        hipLaunchKernelGGL(tau_from_minima_kernel<2>, grid, block, 0, s, gm, G, rank, nq, tau, rt);
    } else if (G <= 256) {
        hipLaunchKernelGGL(tau_from_minima_kernel<4>, grid, block, 0, s, gm, G, rank, nq, tau, rt);
    } else {
        hipLaunchKernelGGL(tau_from_minima_kernel<8>, grid, block, 0, s, gm, G, rank, nq, tau, rt);
    }
}

template <typename S>
static void launch_select_rows_t(const S *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                                 int64_t col_base, unsigned long long *running, bool fresh, hipStream_t s)
{
    if (nrows == 0) {
        return;
    }
    IXA_REQUIRE(ksel >= 1 && ksel <= kSelectMaxK, kErrInvalidParam, "selection size %d out of range [1, %d]", ksel,
                kSelectMaxK);
    const int cap = wave_pool_capacity(ksel);
    // four scanning wavefronts when their pools and the merge fit LDS, else two, else one
    int active = 4;
    while (active > 1 && (size_t)select_region_keys(active, cap, running ? ksel : 0) * sizeof(key_t) + 64 > 160 * 1024) {
        active >>= 1;
    }
    size_t smem = (size_t)select_region_keys(active, cap, running ? ksel : 0) * sizeof(key_t) + 64;
    IXA_REQUIRE(smem <= 160 * 1024, kErrInvalidParam, "selection size %d needs %zu bytes of LDS", ksel, smem);
    const bool vec4 = ld % 4 == 0 && reinterpret_cast<uintptr_t>(scores) % 16 == 0;
    // measured: the register kernel wins on rows of up to a few segments (16384 columns: 0.17 ms against
    // 0.27 ms for 10000 rows, ksel 88), the streaming kernel on rows of hundreds of thousands of columns
    if (vec4 && ksel <= kSelRegMaxK && nc >= 2048 && nc <= 6 * kSelRegSeg) {
        smem = std::max(smem, (size_t)(kSelRegCap + 2 + kSelRegMaxK + 4 * kSelRegStage) * sizeof(key_t) + 4 * 64 * 4 * 4 + 64);
        // groups per lane: ksel / (256 G) stays near 1/3
        auto kern = ksel <= 96 ? select_rows_reg_kernel<S, 1>
                               : (ksel <= 192 ? select_rows_reg_kernel<S, 2> : select_rows_reg_kernel<S, 4>);
        hipLaunchKernelGGL(kern, dim3((unsigned)nrows), dim3(256), smem, s, scores, ld, nc, ksel, cap, out_idx,
                           col_base, running, fresh);
        return;
    }
    auto kern = active == 4 ? select_rows_kernel<S, 4> : (active == 2 ? select_rows_kernel<S, 2> : select_rows_kernel<S, 1>);
    require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    hipLaunchKernelGGL(kern, dim3((unsigned)nrows), dim3(256), smem, s, scores, ld, nc, ksel, cap, out_idx, col_base,
                       running, fresh);
}

void launch_select_rows(const float *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                        int64_t col_base, unsigned long long *running, hipStream_t s, bool fresh)
{
    launch_select_rows_t<float>(scores, nrows, ld, nc, ksel, out_idx, col_base, running, fresh, s);
}

void launch_select_rows_i32(const int32_t *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                            int64_t col_base, unsigned long long *running, hipStream_t s, bool fresh)
{
    launch_select_rows_t<int32_t>(scores, nrows, ld, nc, ksel, out_idx, col_base, running, fresh, s);
}

// ------------------------------------------------------------------------------------------------
// Exact re-evaluation.  Each lane recomputes ONE (query, candidate) score in the canonical order
// (dot product left to right, no FMA, then (|q|^2 + |c|^2) - g - g), the candidates of a query are
// sorted by (score, centroid id) and the best `nout` are written.  Because the MFMA pass only has
// to deliver a superset of the true winners, the result equals the scalar arithmetic bit for bit.
// A workgroup of 256 lanes serves 256 / P queries, P = padded candidate count (power of two).
template <bool VEC4>
__global__ __launch_bounds__(256) void refine_kernel(const float *__restrict__ Q, int64_t nq,
                                                     const float *__restrict__ C, int d,
                                                     const float *__restrict__ qn, const float *__restrict__ cn,
                                                     int metric, const int32_t *__restrict__ cand, int ncand, int P,
                                                     int nout, int out_stride, int32_t *__restrict__ out_ids,
                                                     float *__restrict__ out_dist)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    key_t *keys = reinterpret_cast<key_t *>(smem_raw);
    const int tid = threadIdx.x;
    const int rows_per_block = P >= 256 ? 1 : 256 / P;
    const int total = rows_per_block * P;  // >= 256, power of two
    for (int e = tid; e < total; e += 256) {
        const int sub = e / P, t = e - sub * P;
        const int64_t row = (int64_t)blockIdx.x * rows_per_block + sub;
        key_t key = kEmptyKey;
        if (row < nq && t < ncand) {
            const int32_t c = cand[row * ncand + t];
            if (c >= 0) {
                const float *q = Q + row * d;
                const float *cv = C + (int64_t)c * d;
                float g = 0.f;
                if (VEC4) {
#pragma unroll 8
                    for (int j = 0; j < d; j += 4) {
                        float4 a = *reinterpret_cast<const float4 *>(q + j);
                        float4 b = *reinterpret_cast<const float4 *>(cv + j);
                        g = __fadd_rn(g, __fmul_rn(a.x, b.x));
                        g = __fadd_rn(g, __fmul_rn(a.y, b.y));
                        g = __fadd_rn(g, __fmul_rn(a.z, b.z));
                        g = __fadd_rn(g, __fmul_rn(a.w, b.w));
                    }
                } else {
                    for (int j = 0; j < d; j++) {
                        g = __fadd_rn(g, __fmul_rn(q[j], cv[j]));
                    }
                }
                float v;
                if (metric == kMetricL2) {
                    v = __fadd_rn(qn[row], cn[c]);
                    v = __fsub_rn(v, g);
                    v = __fsub_rn(v, g);
                } else {
                    v = -g;
                }
                key = make_key(v, (uint32_t)c);
            }
        }
        keys[e] = key;
    }
    // segmented bitonic sort: every P-aligned segment ascending
    for (int size = 2; size <= P; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = tid; t < (total >> 1); t += 256) {
                int i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                int j = i + stride;
                bool up = ((i & (P - 1)) & size) == 0;
                key_t a = keys[i], b = keys[j];
                if ((a > b) == up) {
                    keys[i] = b;
                    keys[j] = a;
                }
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < rows_per_block * out_stride; e += 256) {
        const int sub = e / out_stride, t = e - sub * out_stride;
        const int64_t row = (int64_t)blockIdx.x * rows_per_block + sub;
        if (row >= nq) {
            continue;
        }
        key_t kk = t < nout ? keys[sub * P + t] : kEmptyKey;
        const bool ok = kk != kEmptyKey;
        out_ids[row * out_stride + t] = ok ? (int32_t)key_index(kk) : -1;
        if (out_dist) {
            float v = key_score(kk);
            const float pad = metric == kMetricL2 ? 3.402823466e+38f : -3.402823466e+38f;
            out_dist[row * out_stride + t] = ok ? (metric == kMetricL2 ? v : -v) : pad;
        }
    }
}

// Exact selection of the best `nout` candidates as a SET, touching only the candidates that the
// approximate scores cannot decide.  `running` holds, per query, ncand keys sorted by approximate
// score s, each within err = err_scale * |q| * cmax + round_scale * (|q| + cmax)^2 of the canonical score e.  With T = s at rank
// nout: a candidate with s < T - 2 err is certainly among the nout best (fewer than nout others have
// s < T, and only those can have e below its e < T - err); one with s > T + 2 err certainly is not
// (the nout candidates with s <= T all have e <= T + err).  Only the candidates in between are
// re-evaluated in the canonical scalar arithmetic and ranked by (e, id); the best
// nout - |certain| of them complete the set.  Centroids outside the list have s >= s_last, so the
// set is proven complete when s_last > T + 2 err; otherwise the query is appended to the list
// flag[1 + flag[0]++] and the caller must use another plan for it.  One wavefront per query; out_ids gets nout ids in no particular order.
template <bool VEC4>
__global__ __launch_bounds__(256) void refine_boundary_kernel(const float *__restrict__ Q, int64_t nq,
                                                              const float *__restrict__ C, int d,
                                                              const float *__restrict__ qn,
                                                              const float *__restrict__ cn, int metric,
                                                              const key_t *__restrict__ running, int ncand, int nout,
                                                              float cmax, float err_scale, float round_scale,
                                                              int32_t *__restrict__ out_ids, int *__restrict__ flag,
                                                              int complete)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= nq) {
        return;
    }
    key_t *ekeys = reinterpret_cast<key_t *>(smem_raw) + (size_t)wave * ncand;          // exact keys of the undecided
    int32_t *amb = reinterpret_cast<int32_t *>(smem_raw + (size_t)4 * ncand * sizeof(key_t)) + (size_t)wave * ncand;
    const key_t *run = running + row * ncand;
    int32_t *out = out_ids + row * nout;
    const key_t at_rank = run[nout - 1];
    if (at_rank == kEmptyKey) {
        // fewer than nout candidates exist at all: every one of them is in
        for (int i = lane; i < nout; i += kWave) {
            const key_t kk = run[i];
            out[i] = kk == kEmptyKey ? -1 : (int32_t)key_index(kk);
        }
        return;
    }
    const float T = key_score(at_rank);
    const float qlen = sqrtf(qn[row]);
    const float err = err_scale * qlen * cmax + round_scale * (qlen + cmax) * (qlen + cmax);
    const float lo = T - 2.0f * err, hi = T + 2.0f * err;
    const key_t last = run[ncand - 1];
    if (lane == 0 && !complete && last != kEmptyKey && !(key_score(last) > hi)) {   // a list of all rows is complete
        flag[1 + atomicAdd(flag, 1)] = (int)row;   // the list of queries that need another plan
    }
    int n_in = 0, n_amb = 0;
    for (int base = 0; base < ncand; base += kWave) {
        const int i = base + lane;
        const key_t kk = i < ncand ? run[i] : kEmptyKey;
        const float sc = key_score(kk);
        const bool valid = kk != kEmptyKey;
        const bool in = valid && sc < lo;
        const bool und = valid && !in && sc <= hi;
        const unsigned long long m_in = __ballot(in), m_und = __ballot(und);
        const int p_in = __builtin_amdgcn_mbcnt_hi((uint32_t)(m_in >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m_in, 0));
        const int p_und =
            __builtin_amdgcn_mbcnt_hi((uint32_t)(m_und >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m_und, 0));
        if (in) {
            out[n_in + p_in] = (int32_t)key_index(kk);
        }
        if (und) {
            amb[n_amb + p_und] = (int32_t)key_index(kk);
        }
        n_in += __popcll(m_in);
        n_amb += __popcll(m_und);
    }
    wave_lds_fence();
    const float *q = Q + row * d;
    for (int j = lane; j < n_amb; j += kWave) {
        const int32_t c = amb[j];
        const float *cv = C + (int64_t)c * d;
        float g = 0.f;
        if (VEC4) {
#pragma unroll 8
            for (int t = 0; t < d; t += 4) {
                const float4 a = *reinterpret_cast<const float4 *>(q + t);
                const float4 b = *reinterpret_cast<const float4 *>(cv + t);
                g = __fadd_rn(g, __fmul_rn(a.x, b.x));
                g = __fadd_rn(g, __fmul_rn(a.y, b.y));
                g = __fadd_rn(g, __fmul_rn(a.z, b.z));
                g = __fadd_rn(g, __fmul_rn(a.w, b.w));
            }
        } else {
            for (int t = 0; t < d; t++) {
                g = __fadd_rn(g, __fmul_rn(q[t], cv[t]));
            }
        }
        float v;
        if (metric == kMetricL2) {
            v = __fadd_rn(qn[row], cn[c]);
            v = __fsub_rn(v, g);
            v = __fsub_rn(v, g);
        } else {
            v = -g;
        }
        ekeys[j] = make_key(v, (uint32_t)c);
    }
    wave_lds_fence();
    const int need = nout - n_in;   // >= 1: the candidate at rank nout is itself undecided
    for (int j = lane; j < n_amb; j += kWave) {
        const key_t mine = ekeys[j];
        int rank = 0;
        for (int t = 0; t < n_amb; t++) {
            rank += ekeys[t] < mine ? 1 : 0;
        }
        if (rank < need) {
            out[n_in + rank] = (int32_t)key_index(mine);
        }
    }
}

void launch_refine_boundary(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn,
                            int metric, const unsigned long long *running, int ncand, int nout, float cmax,
                            float err_scale, float round_scale, int32_t *out_ids, int *flag, bool complete,
                            hipStream_t s)
{
    if (nq == 0) {
        return;
    }
    IXA_REQUIRE(ncand >= 1 && ncand <= 3072 && nout >= 1 && nout <= ncand, kErrInvalidParam,
                "refine candidate count %d out of range [1, 3072]", ncand);
    const size_t smem = (size_t)4 * ncand * (sizeof(key_t) + sizeof(int32_t));
    const bool vec4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(Q) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    auto kern = vec4 ? refine_boundary_kernel<true> : refine_boundary_kernel<false>;
    require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    hipLaunchKernelGGL(kern, dim3((unsigned)((nq + 3) / 4)), dim3(256), smem, s, Q, nq, C, d, qn, cn, metric, running,
                       ncand, nout, cmax, err_scale, round_scale, out_ids, flag, complete ? 1 : 0);
}

// The boundary refinement above straight from the records of a record-mode score launch over the whole
// base (see launch_fold_records), without a sorted list in between: one wavefront per query compacts the
// recorded scores at or below tau into LDS, finds T = the approximate score at rank nout by bisection
// over the ordered score bits (the scores in registers), classifies against T -+ 2 err and re-evaluates
// the undecided as above.  The records hold EVERY centroid whose approximate score is at or below tau,
// so the set is proven complete when tau > T + 2 err -- whatever tau was derived from.  A query without
// proof (that, dropped records, more scores than the wave's 64 E places, more undecided candidates than
// amb_cap) is appended to flag[1 + flag[0]++] for the caller's exact plan, and its nout ids are all -1.
template <bool VEC4, int E>
__global__ __launch_bounds__(256) void fold_refine_boundary_kernel(
    const float *__restrict__ Q, int64_t nq, const float *__restrict__ C, int d, const float *__restrict__ qn,
    const float *__restrict__ cn, int metric, ScoreFilter<float> flt, int amb_cap, int nout, float cmax,
    float err_scale, float round_scale, int32_t *__restrict__ out_ids, int *__restrict__ flag, int64_t row_base, bool raw)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int capk = 64 * E;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= nq) {
        return;
    }
    const size_t per_wave = (size_t)capk * sizeof(key_t) + (size_t)amb_cap * (sizeof(key_t) + sizeof(int32_t));
    key_t *keys = reinterpret_cast<key_t *>(smem_raw + wave * per_wave);
    key_t *ekeys = keys + capk;
    int32_t *amb = reinterpret_cast<int32_t *>(ekeys + amb_cap);
    int32_t *out = out_ids + row * nout;
    const float tau = flt.tau[row];
    int nrec = flt.cnt[row];
    bool fail = nrec > flt.cap;   // wave-uniform: records were dropped
    nrec = nrec > flt.cap ? flt.cap : nrec;
    nrec = __builtin_amdgcn_readfirstlane(nrec);
    const float qnorm = qn[row];
    // ---- every recorded score at or below tau, compacted; eight loads of 64 records in flight at a time
    int n = 0;
    const unsigned char *records = reinterpret_cast<const unsigned char *>(flt.cand) + (int64_t)row * flt.cap * 32;
    constexpr int kBatch = 8;
    for (int base = 0; base < nrec; base += kBatch * kWave) {
        float4 sc[kBatch];
        uint32_t col[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            const int r = base + b * kWave + lane;
            sc[b] = make_float4(0.f, 0.f, 0.f, 0.f);
            col[b] = 0;
            if (r < nrec) {
                sc[b] = *reinterpret_cast<const float4 *>(records + (int64_t)r * 32);
                col[b] = *reinterpret_cast<const uint32_t *>(records + (int64_t)r * 32 + 16);
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            if (base + b * kWave >= nrec) {
                break;   // wave-uniform
            }
            const int r = base + b * kWave + lane;
            float v[4] = {sc[b].x, sc[b].y, sc[b].z, sc[b].w};
            record_scores(v, raw, metric, qnorm, cn, col[b]);   // lanes past nrec hold column 0: a valid address
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const bool pass = r < nrec && v[t] <= tau;
                const unsigned long long m = __ballot(pass);
                if (m) {
                    const int pos = n + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                                                       __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
                    if (pass && pos < capk) {
                        keys[pos] = make_key(v[t], col[b] + (uint32_t)t);
                    }
                    n += __popcll(m);
                }
            }
        }
    }
    if (lane == 0) {
        flt.cnt[row] = 0;   // the next launch's records start at zero
    }
    fail = fail || n > capk || n < nout;
    wave_lds_fence();
    float lo = 0.f, hi = 0.f;
    if (!fail) {
        // ordered bits of the score at rank nout: the largest value with fewer than nout scores below it,
        // built from the top bit down
        uint32_t u[E];
#pragma unroll
        for (int e = 0; e < E; e++) {
            const int i = e * kWave + lane;
            u[e] = i < n ? (uint32_t)(keys[i] >> 32) : 0xffffffffu;
        }
        uint32_t p = 0;
        for (int bit = 31; bit >= 0; bit--) {
            const uint32_t c = p | (1u << bit);
            int below = 0;
#pragma unroll
            for (int e = 0; e < E; e++) {
                below += __popcll(__ballot(u[e] < c));
            }
            p = below < nout ? c : p;
        }
        const float T = unordered_bits(p);
        const float qlen = sqrtf(qnorm);
        const float err = err_scale * qlen * cmax + round_scale * (qlen + cmax) * (qlen + cmax);
        lo = T - 2.0f * err;
        hi = T + 2.0f * err;
        fail = !(tau > hi);
    }
    int n_in = 0, n_amb = 0;
    if (!fail) {
        for (int base = 0; base < n; base += kWave) {
            const int i = base + lane;
            const key_t kk = i < n ? keys[i] : kEmptyKey;
            const float sc = key_score(kk);
            const bool in = i < n && sc < lo;
            const bool und = i < n && !in && sc <= hi;
            const unsigned long long m_in = __ballot(in), m_und = __ballot(und);
            const int p_in =
                __builtin_amdgcn_mbcnt_hi((uint32_t)(m_in >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m_in, 0));
            const int p_und =
                __builtin_amdgcn_mbcnt_hi((uint32_t)(m_und >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m_und, 0));
            if (in) {
                out[n_in + p_in] = (int32_t)key_index(kk);   // fewer than nout scores lie below T
            }
            if (und && n_amb + p_und < amb_cap) {
                amb[n_amb + p_und] = (int32_t)key_index(kk);
            }
            n_in += __popcll(m_in);
            n_amb += __popcll(m_und);
        }
        fail = n_amb > amb_cap;
    }
    if (fail) {
        // the row's ids must not stay what the memory happened to hold: work queued behind this launch (the scan
        // of a search) may read them before the caller's exact plan has replaced them, and -1 is "no list" there
        for (int i = lane; i < nout; i += kWave) {
            out[i] = -1;
        }
        if (lane == 0) {
            flag[1 + atomicAdd(flag, 1)] = (int)(row_base + row);   // the list of queries that need another plan
        }
        return;
    }
    wave_lds_fence();
    const float *q = Q + row * d;
    for (int j = lane; j < n_amb; j += kWave) {
        const int32_t c = amb[j];
        const float *cv = C + (int64_t)c * d;
        float g = 0.f;
        if (VEC4) {
#pragma unroll 8
            for (int t = 0; t < d; t += 4) {
                const float4 a = *reinterpret_cast<const float4 *>(q + t);
                const float4 b = *reinterpret_cast<const float4 *>(cv + t);
                g = __fadd_rn(g, __fmul_rn(a.x, b.x));
                g = __fadd_rn(g, __fmul_rn(a.y, b.y));
                g = __fadd_rn(g, __fmul_rn(a.z, b.z));
                g = __fadd_rn(g, __fmul_rn(a.w, b.w));
            }
        } else {
            for (int t = 0; t < d; t++) {
                g = __fadd_rn(g, __fmul_rn(q[t], cv[t]));
            }
        }
        float v;
        if (metric == kMetricL2) {
            v = __fadd_rn(qnorm, cn[c]);
            v = __fsub_rn(v, g);
            v = __fsub_rn(v, g);
        } else {
            v = -g;
        }
        ekeys[j] = make_key(v, (uint32_t)c);
    }
    wave_lds_fence();
    const int need = nout - n_in;   // >= 1: the candidate at rank nout is itself undecided
    for (int j = lane; j < n_amb; j += kWave) {
        const key_t mine = ekeys[j];
        int rank = 0;
        for (int t = 0; t < n_amb; t++) {
            rank += ekeys[t] < mine ? 1 : 0;
        }
        if (rank < need) {
            out[n_in + rank] = (int32_t)key_index(mine);
        }
    }
}

template <bool VEC4>
static void launch_fold_refine_boundary_t(const float *Q, int64_t nq, const float *C, int d, const float *qn,
                                          const float *cn, int metric, ScoreFilter<float> flt, int capk, int nout,
                                          float cmax, float err_scale, float round_scale, int32_t *out_ids, int *flag,
                                          int64_t row_base, bool raw, hipStream_t s)
{
    const int amb_cap = 128;
    const int E = capk <= 256 ? 4 : (capk <= 512 ? 8 : (capk <= 1024 ? 16 : 32));
    const size_t smem = (size_t)4 * ((size_t)64 * E * sizeof(key_t) + (size_t)amb_cap * (sizeof(key_t) + sizeof(int32_t)));
    auto kern = E == 4 ? fold_refine_boundary_kernel<VEC4, 4>
                       : (E == 8 ? fold_refine_boundary_kernel<VEC4, 8>
                                 : (E == 16 ? fold_refine_boundary_kernel<VEC4, 16> : fold_refine_boundary_kernel<VEC4, 32>));
    require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    hipLaunchKernelGGL(kern, dim3((unsigned)((nq + 3) / 4)), dim3(256), smem, s, Q, nq, C, d, qn, cn, metric, flt,
                       amb_cap, nout, cmax, err_scale, round_scale, out_ids, flag, row_base, raw);
}

void launch_fold_refine_boundary(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn,
                                 int metric, ScoreFilter<float> flt, int capk, int nout, float cmax, float err_scale,
                                 float round_scale, int32_t *out_ids, int *flag, int64_t row_base, hipStream_t s,
                                 bool raw)
{
    if (nq == 0) {
        return;
    }
    IXA_REQUIRE(nout >= 1 && capk >= nout && capk <= 2048, kErrInner, "fold refine of %d from %d keys", nout, capk);
    IXA_REQUIRE(!raw || reinterpret_cast<uintptr_t>(cn) % 16 == 0, kErrInner, "raw records need aligned norms");
    const bool vec4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(Q) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    if (vec4) {
        launch_fold_refine_boundary_t<true>(Q, nq, C, d, qn, cn, metric, flt, capk, nout, cmax, err_scale, round_scale,
                                            out_ids, flag, row_base, raw, s);
    } else {
        launch_fold_refine_boundary_t<false>(Q, nq, C, d, qn, cn, metric, flt, capk, nout, cmax, err_scale,
                                             round_scale, out_ids, flag, row_base, raw, s);
    }
}

// Canonical scores of whole rows: out[row * ldo + col] for every centroid, one lane per score, in the
// arithmetic of the refinement kernels (dot product left to right, no FMA).  The plan of last resort
// for queries whose approximate candidate lists cannot be proven complete: slow, exact by construction.
// Without row norms (qn == nullptr, L2) every lane adds up its row's squares beside the dot product, in the
// order of sqnorm_rows_kernel, so the scores are the same bits and a small search saves that launch.
template <bool VEC4>
__global__ __launch_bounds__(256) void canonical_scores_kernel(const float *__restrict__ Q, int64_t nq,
                                                               const float *__restrict__ C, int64_t nc, int d,
                                                               const float *__restrict__ qn,
                                                               const float *__restrict__ cn, int metric,
                                                               float *__restrict__ out, int64_t ldo)
{
    const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    if (col >= nc) {
        return;
    }
    const float *q = Q + row * d;
    const float *cv = C + col * d;
    const bool own_norm = qn == nullptr && metric == kMetricL2;
    float g = 0.f, qq = 0.f;
    if (VEC4) {
#pragma unroll 4
        for (int t = 0; t < d; t += 4) {
            const float4 a = *reinterpret_cast<const float4 *>(q + t);
            const float4 b = *reinterpret_cast<const float4 *>(cv + t);
            g = __fadd_rn(g, __fmul_rn(a.x, b.x));
            g = __fadd_rn(g, __fmul_rn(a.y, b.y));
            g = __fadd_rn(g, __fmul_rn(a.z, b.z));
            g = __fadd_rn(g, __fmul_rn(a.w, b.w));
            if (own_norm) {
                qq = __fadd_rn(qq, __fmul_rn(a.x, a.x));
                qq = __fadd_rn(qq, __fmul_rn(a.y, a.y));
                qq = __fadd_rn(qq, __fmul_rn(a.z, a.z));
                qq = __fadd_rn(qq, __fmul_rn(a.w, a.w));
            }
        }
    } else {
        for (int t = 0; t < d; t++) {
            g = __fadd_rn(g, __fmul_rn(q[t], cv[t]));
            if (own_norm) {
                qq = __fadd_rn(qq, __fmul_rn(q[t], q[t]));
            }
        }
    }
    float v;
    if (metric == kMetricL2) {
        v = __fadd_rn(own_norm ? qq : qn[row], cn[col]);
        v = __fsub_rn(v, g);
        v = __fsub_rn(v, g);
    } else {
        v = -g;
    }
    out[row * ldo + col] = v;
}

void launch_canonical_scores(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                             const float *cn, int metric, float *out, int64_t ldo, hipStream_t s)
{
    if (nq == 0 || nc == 0) {
        return;
    }
    IXA_REQUIRE(nq <= 65535, kErrInner, "canonical score launch of %ld rows", (long)nq);
    const bool vec4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(Q) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    const dim3 grid((unsigned)((nc + 255) / 256), (unsigned)nq);
    if (vec4) {
        hipLaunchKernelGGL(canonical_scores_kernel<true>, grid, dim3(256), 0, s, Q, nq, C, nc, d, qn, cn, metric, out, ldo);
    } else {
        hipLaunchKernelGGL(canonical_scores_kernel<false>, grid, dim3(256), 0, s, Q, nq, C, nc, d, qn, cn, metric, out, ldo);
    }
}

// dist[row * k + t] = the score at column idx[row * k + t], as the public distance (inner products are
// stored negated in the score matrix); (+-FLT_MAX where idx is -1).
__global__ __launch_bounds__(256) void gather_scores_kernel(const float *__restrict__ scores, int64_t ld,
                                                            const int32_t *__restrict__ idx, int64_t n, int k, int metric,
                                                            float *__restrict__ dist)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n * k) {
        return;
    }
    const int32_t c = idx[e];
    const float pad = metric == kMetricL2 ? 3.402823466e+38f : -3.402823466e+38f;
    const float v = c >= 0 ? scores[(e / k) * ld + c] : 0.f;
    dist[e] = c >= 0 ? (metric == kMetricL2 ? v : -v) : pad;
}

void launch_gather_scores(const float *scores, int64_t ld, const int32_t *idx, int64_t n, int k, int metric, float *dist,
                          hipStream_t s)
{
    if (n * k > 0) {
        hipLaunchKernelGGL(gather_scores_kernel, dim3((unsigned)((n * k + 255) / 256)), dim3(256), 0, s, scores, ld, idx,
                           n, k, metric, dist);
    }
}

void launch_refine(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn, int metric,
                   const int32_t *cand, int ncand, int nout, int out_stride, int32_t *out_ids, float *out_dist,
                   hipStream_t s)
{
    if (nq == 0) {
        return;
    }
    IXA_REQUIRE(ncand >= 1 && ncand <= 4096 && nout <= ncand && out_stride >= nout, kErrInvalidParam,
                "refine candidate count %d out of range [1, 4096]", ncand);
    const int P = pow2_ceil(ncand < 2 ? 2 : ncand);
    const int rows_per_block = P >= 256 ? 1 : 256 / P;
    const unsigned grid = (unsigned)((nq + rows_per_block - 1) / rows_per_block);
    const size_t smem = (size_t)rows_per_block * P * sizeof(key_t);
    const bool vec4 = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(Q) % 16 == 0) &&
                      (reinterpret_cast<uintptr_t>(C) % 16 == 0);
    if (vec4) {
        hipLaunchKernelGGL(refine_kernel<true>, dim3(grid), dim3(256), smem, s, Q, nq, C, d, qn, cn, metric, cand,
                           ncand, P, nout, out_stride, out_ids, out_dist);
    } else {
        hipLaunchKernelGGL(refine_kernel<false>, dim3(grid), dim3(256), smem, s, Q, nq, C, d, qn, cn, metric, cand,
                           ncand, P, nout, out_stride, out_ids, out_dist);
    }
}

}  // namespace ixa
