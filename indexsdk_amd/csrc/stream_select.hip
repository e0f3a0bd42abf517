// Host driver of the streaming brute-force selection (see stream_select.h).
#include "stream_select.h"

#include <algorithm>
#include <cmath>

#include "flat_i8.h"
#include "topk.h"

namespace ixa {

namespace {

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

// tau[row] = score of the last running key of the row, or the worst score while the row is not full.
template <typename S>
__global__ __launch_bounds__(256) void tau_from_running_kernel(const key_t *__restrict__ running, int k, int64_t n,
                                                               S *__restrict__ tau)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const key_t last = running[i * k + (k - 1)];
        tau[i] = last == kEmptyKey ? ScoreOps<S>::worst() : key_score_as<S>(last);
    }
}

__global__ __launch_bounds__(256) void keys_to_idx_kernel(const key_t *__restrict__ keys, int64_t n,
                                                          int32_t *__restrict__ out)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        out[i] = keys[i] == kEmptyKey ? -1 : (int32_t)key_index(keys[i]);
    }
}

// thr[i] = min(tau[i], kI8MaxBound) - qn[i]: a bound above every possible distance (a row that is not full yet has
// the worst score for one) admits every row either way, and the score kernels rely on the smaller number
__global__ __launch_bounds__(256) void threshold_i32_kernel(const int32_t *__restrict__ tau,
                                                            const int32_t *__restrict__ qn, int64_t n,
                                                            int32_t *__restrict__ thr)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        thr[i] = min(tau[i], kI8MaxBound) - qn[i];   // qn >= 0: no overflow
    }
}

// One thread per (score row, mask byte): the eight base rows of the byte, those inside the stretch.
template <typename S>
__global__ __launch_bounds__(256) void apply_mask_kernel(S *__restrict__ scores, int64_t nq, int64_t ld, int64_t nc,
                                                         const uint8_t *__restrict__ mask, int64_t stride,
                                                         const int64_t *__restrict__ row_map, int64_t col0,
                                                         int64_t first_byte, int64_t nbytes)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nq * nbytes) {
        return;
    }
    const int64_t r = i / nbytes, b = first_byte + i % nbytes;
    const uint8_t m = mask[(row_map ? row_map[r] : r) * stride + b];
    if (m == 0xff) {
        return;
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int64_t c = (b << 3) + t - col0;
        if (c >= 0 && c < nc && !((m >> t) & 1)) {
            scores[r * ld + c] = ScoreOps<S>::worst();
        }
    }
}

template <typename S>
void apply_mask(S *scores, int64_t nq, int64_t ld, int64_t nc, const uint8_t *mask, int64_t stride,
                const int64_t *row_map, int64_t col0, hipStream_t s)
{
    if (nq <= 0 || nc <= 0) {
        return;
    }
    const int64_t first_byte = col0 >> 3, nbytes = ((col0 + nc + 7) >> 3) - first_byte;
    IXA_REQUIRE(mask != nullptr && ((col0 + nc + 7) >> 3) <= stride, kErrInner,
                "mask rows of %ld bytes do not cover base rows up to %ld", (long)stride, (long)(col0 + nc));
    hipLaunchKernelGGL(apply_mask_kernel<S>, dim3(blocks_for(nq * nbytes)), dim3(256), 0, s, scores, nq, ld, nc, mask,
                       stride, row_map, col0, first_byte, nbytes);
}

template <typename S>
__global__ __launch_bounds__(256) void drop_worst_keys_kernel(key_t *__restrict__ keys, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const key_t kk = keys[i];
        if (kk != kEmptyKey && key_score_as<S>(kk) == ScoreOps<S>::worst()) {
            keys[i] = kEmptyKey;
        }
    }
}

struct F32Ops {
    using T = float;
    using S = float;
    static constexpr int64_t kMinChunk = 1;   // its score launchers serve any chunk of base rows
    static constexpr int64_t kSeedRows = 2048, kMaxGrowth = 1 << 20;
    const float *qn, *bn;
    int metric;
    const S *threshold(StreamSelectWorkspace<S> &, int64_t, int64_t, hipStream_t) const { return nullptr; }
    void scores(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, S *out, int64_t ldo,
                hipStream_t s) const
    {
        launch_score_tiles(Q, nq, B + b0 * d, nb, d, qn + q0, bn + b0, metric, out, ldo, s);
    }
    void filtered(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, ScoreFilter<S> flt,
                  hipStream_t s) const
    {
        launch_score_tiles_filtered(Q, nq, B + b0 * d, nb, d, qn + q0, bn + b0, metric, flt, s);
    }
    void select(const S *sc, int64_t nq, int64_t ld, int64_t nc, int k, int64_t base, key_t *run, bool fresh,
                hipStream_t s) const
    {
        launch_select_rows(sc, nq, ld, nc, k, nullptr, base, run, s, fresh);
    }
    static constexpr bool kMergeKeepsThreshold = false;
    void merge(key_t *run, int k, ScoreFilter<S> flt, S *tau, int64_t nq, int64_t, int *ovf, hipStream_t s) const
    {
        launch_merge_candidates(run, k, flt, tau, nq, ovf, s);
    }
};

struct Bf16Ops {
    using T = uint16_t;
    using S = float;
    static constexpr int64_t kMinChunk = 2048;   // the ring kernel is the only one for split operands
    static constexpr int64_t kSeedRows = 2048, kMaxGrowth = 1 << 20;
    const float *qn, *bn;
    int metric;
    const S *threshold(StreamSelectWorkspace<S> &, int64_t, int64_t, hipStream_t) const { return nullptr; }
    void scores(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, S *out, int64_t ldo,
                hipStream_t s) const
    {
        const bool ok = launch_score_ring_bf16(Q, nq, B + b0 * d, nb, d, qn + q0, bn + b0, metric, out, ldo, false,
                                               ScoreFilter<float>{}, s);
        IXA_REQUIRE(ok, kErrInner, "bf16 score kernel rejected a shape it had accepted");
    }
    void filtered(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, ScoreFilter<S> flt,
                  hipStream_t s) const
    {
        const bool ok = launch_score_ring_bf16(Q, nq, B + b0 * d, nb, d, qn + q0, bn + b0, metric, nullptr, 0, true, flt, s);
        IXA_REQUIRE(ok, kErrInner, "bf16 score kernel rejected a shape it had accepted");
    }
    void select(const S *sc, int64_t nq, int64_t ld, int64_t nc, int k, int64_t base, key_t *run, bool fresh,
                hipStream_t s) const
    {
        launch_select_rows(sc, nq, ld, nc, k, nullptr, base, run, s, fresh);
    }
    static constexpr bool kMergeKeepsThreshold = false;
    void merge(key_t *run, int k, ScoreFilter<S> flt, S *tau, int64_t nq, int64_t, int *ovf, hipStream_t s) const
    {
        launch_merge_candidates(run, k, flt, tau, nq, ovf, s);
    }
};

// B is the base in matrix-core order (flat_i8.h) and bn its norms, padded to whole tiles: a stretch of the base is
// named by its rows, never by a pointer into it
struct I8Ops {
    using T = int8_t;
    using S = int32_t;
    static constexpr int64_t kMinChunk = 1;
    // A launch of the resident-query kernel costs little and its bound-filtered epilogue is cheapest when few scores
    // pass, so the bound is tightened often: a longer seed stretch (a bound from 8192 rows admits a quarter of what
    // one from 2048 does) and chunks that only double what has been seen (10M x 512, 2048 queries, k 100, same box:
    // seed 2048 and chunks of 5 x seen 8.91 ms per search; 8192 and 5 x: 8.80; 8192 and 3 x: 8.54; 8192 and 2 x: 8.47)
    static constexpr int64_t kSeedRows = 8192, kMaxGrowth = 2;
    const int32_t *qn, *bn;
    const S *threshold(StreamSelectWorkspace<S> &ws, int64_t q0, int64_t nq, hipStream_t s) const
    {
        hipLaunchKernelGGL(threshold_i32_kernel, dim3(blocks_for(nq)), dim3(256), 0, s, ws.tau.data() + q0, qn + q0, nq,
                           ws.thr.data() + q0);
        return ws.thr.data() + q0;
    }
    void scores(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, S *out, int64_t ldo,
                hipStream_t s) const
    {
        launch_i8_scores_stored(Q, nq, B, d, qn + q0, bn, b0, b0 + nb, out, ldo, s);
    }
    void filtered(const T *Q, int64_t nq, int64_t q0, const T *B, int64_t nb, int64_t b0, int d, ScoreFilter<S> flt,
                  hipStream_t s) const
    {
        launch_i8_scores_filtered(Q, nq, B, d, qn + q0, bn, b0, b0 + nb, flt, s);
    }
    void select(const S *sc, int64_t nq, int64_t ld, int64_t nc, int k, int64_t base, key_t *run, bool fresh,
                hipStream_t s) const
    {
        launch_select_rows_i32(sc, nq, ld, nc, k, nullptr, base, run, s, fresh);
    }
    // the merge writes the next launch's thresholds along with the new bounds
    static constexpr bool kMergeKeepsThreshold = true;
    void merge(key_t *run, int k, ScoreFilter<S> flt, S *tau, int64_t nq, int64_t q0, int *ovf, hipStream_t s) const
    {
        launch_merge_candidates_i32(run, k, flt, tau, nq, ovf, s, const_cast<S *>(flt.thr), qn + q0, kI8MaxBound);
    }
};

template <typename Ops>
int stream_select(const Ops &ops, const typename Ops::T *Q, int64_t nq_total, const typename Ops::T *B, int64_t nb_total,
                  int d, int ncand, key_t *running, StreamSelectWorkspace<typename Ops::S> &ws, int64_t scratch_bytes,
                  hipStream_t s, const uint8_t *mask = nullptr, int64_t mask_stride = 0)
{
    using S = typename Ops::S;
    if (nq_total == 0) {
        return 0;
    }
    if (nb_total == 0) {   // no chunk will start the running keys
        IXA_HIP(hipMemsetAsync(running, 0xff, (size_t)nq_total * ncand * sizeof(key_t), s));
        return 0;
    }
    int64_t qb = std::min<int64_t>(round_up(nq_total, 128), 16384);
    if (scratch_bytes / (qb * (int64_t)sizeof(S)) < Ops::kMinChunk) {
        // a small scratch: fewer query rows per block rather than chunks narrower than the kernel serves
        qb = std::max<int64_t>(128, scratch_bytes / (Ops::kMinChunk * (int64_t)sizeof(S)) / 128 * 128);
    }
    int64_t nb = scratch_bytes / (qb * (int64_t)sizeof(S));
    nb = std::max<int64_t>(128, nb / 128 * 128);
    nb = std::min<int64_t>(nb, round_up(std::max<int64_t>(nb_total, 1), 128));
    const int cap = pow2_ceil((int)std::max<int64_t>(1024, 16 * (int64_t)ncand));
    const int64_t seed_rows = std::min<int64_t>(nb_total, std::max<int64_t>(Ops::kSeedRows, 16 * (int64_t)ncand));
    // when the whole score matrix of a query block fits the scratch, one materialised pass is the
    // cheapest plan (measured on the IVFPQ coarse stage: 16384 centroids); the filtered plan is for
    // long bases
    // (a masked search materialises every stretch: the mask is applied to the stored scores)
    bool can_fuse = mask == nullptr && nb_total > nb && nb_total >= 4 * seed_rows &&
                    pow2_ceil(ncand + cap) * sizeof(key_t) <= 160 * 1024;
    if (can_fuse && qb * (int64_t)cap * (int64_t)sizeof(key_t) > scratch_bytes) {
        // the candidate buffers of a query block count against the scratch budget too: a narrower block
        qb = std::max<int64_t>(128, scratch_bytes / ((int64_t)cap * (int64_t)sizeof(key_t)) / 128 * 128);
        nb = scratch_bytes / (qb * (int64_t)sizeof(S));
        nb = std::max<int64_t>(128, nb / 128 * 128);
        nb = std::min<int64_t>(nb, round_up(std::max<int64_t>(nb_total, 1), 128));
        can_fuse = nb_total > nb;
    }
    // tau is fixed during a chunk, so a chunk admits about ncand * chunk / seen keys per query; keep
    // that expectation below a quarter of the candidate buffer
    const int64_t growth = std::max<int64_t>(2, std::min<int64_t>(Ops::kMaxGrowth, cap / (4 * (int64_t)ncand)));
    if (Ops::kMinChunk > 1) {
        // Dry run of the chunking below (the filtered plan and the materialised one it falls back to): every
        // chunk must be one the score kernel serves, or the caller takes another route.
        const int64_t ld_plan = can_fuse ? std::min(nb, round_up(seed_rows, 128)) : nb;
        bool ok = true;
        auto walk = [&](int64_t head, int64_t width) {
            for (int64_t b0 = 0; b0 < head; b0 += width) {
                ok = ok && std::min(width, head - b0) >= Ops::kMinChunk;
            }
        };
        walk(nb_total, nb);
        if (can_fuse) {
            walk(seed_rows, ld_plan);
            for (int64_t seen = seed_rows; seen < nb_total;) {
                const int64_t nbc = std::min<int64_t>({nb_total - seen, seen * growth, (int64_t)1 << 23});
                ok = ok && nbc >= Ops::kMinChunk;
                seen += nbc;
            }
        }
        if (!ok) {
            return -1;
        }
    }
    // the scratch only has to hold the seeding stretch unless the fallback is taken
    ws.scores.resize((size_t)qb * (can_fuse ? std::min(nb, round_up(seed_rows, 128)) : nb));
    const int64_t ld = can_fuse ? std::min(nb, round_up(seed_rows, 128)) : nb;
    ws.tau.resize((size_t)nq_total);
    ws.thr.resize((size_t)nq_total);
    ws.cnt.resize((size_t)nq_total + 1);
    ws.cnt_zero = false;
    if (can_fuse) {
        ws.filter.resize((size_t)qb * cap);
    }
    if (can_fuse) {   // per-query candidate counters and the overflow flag of the filtered launches
        IXA_HIP(hipMemsetAsync(ws.cnt.data(), 0, ws.cnt.bytes(), s));
    }
    int *overflow = ws.cnt.data() + nq_total;
    int launches = 0;
    bool fused = can_fuse;
    for (int attempt = 0; attempt < 2; attempt++) {
        int64_t ldo = ld;
        if (!fused && can_fuse) {
            ws.scores.resize((size_t)qb * nb);  // fallback: the scratch walks the whole base
            ldo = nb;
        }
        for (int64_t q0 = 0; q0 < nq_total; q0 += qb) {
            const int64_t nq = std::min(qb, nq_total - q0);
            const int64_t head = fused ? seed_rows : nb_total;
            for (int64_t b0 = 0; b0 < head; b0 += ldo) {
                const int64_t nbc = std::min(ldo, head - b0);
                ops.scores(Q + q0 * d, nq, q0, B, nbc, b0, d, ws.scores.data(), ldo, s);
                if (mask) {
                    apply_mask(ws.scores.data(), nq, ldo, nbc, mask + q0 * mask_stride, mask_stride, nullptr, b0, s);
                }
                // the first chunk of a query block starts its running keys (whatever `running` held)
                ops.select(ws.scores.data(), nq, ldo, nbc, ncand, b0, running + q0 * ncand, b0 == 0, s);
                launches++;
            }
            if (!fused) {
                continue;
            }
            hipLaunchKernelGGL(tau_from_running_kernel<S>, dim3(blocks_for(nq)), dim3(256), 0, s,
                               running + q0 * ncand, ncand, nq, ws.tau.data() + q0);
            int64_t seen = head;
            const S *thr = nullptr;
            bool first_chunk = true;
            while (seen < nb_total) {
                const int64_t nbc = std::min<int64_t>({nb_total - seen, seen * growth, (int64_t)1 << 23});
                if (first_chunk || !Ops::kMergeKeepsThreshold) {
                    thr = ops.threshold(ws, q0, nq, s);
                    first_chunk = false;
                }
                ScoreFilter<S> flt{ws.tau.data() + q0, thr, ws.cnt.data() + q0, ws.filter.data(), cap, seen};
                ops.filtered(Q + q0 * d, nq, q0, B, nbc, seen, d, flt, s);
                ops.merge(running + q0 * ncand, ncand, flt, ws.tau.data() + q0, nq, q0, overflow, s);
                launches++;
                seen += nbc;
            }
        }
        if (!fused) {
            break;   // nothing can overflow: no host synchronisation, the caller's stream carries on
        }
        int ovf = 0;
        IXA_HIP(hipMemcpyAsync(&ovf, overflow, sizeof(int), hipMemcpyDeviceToHost, s));
        sync_stream(s);
        if (!ovf) {
            break;
        }
        fused = false;
    }
    return launches;
}

}  // namespace

int stream_select_f32(const float *Q, int64_t nq, const float *B, int64_t nb, int d, const float *qn, const float *bn,
                      int metric, int ncand, unsigned long long *running, StreamSelectWorkspace<float> &ws,
                      int64_t scratch_bytes, hipStream_t s, const uint8_t *mask, int64_t mask_stride)
{
    return stream_select(F32Ops{qn, bn, metric}, Q, nq, B, nb, d, ncand, running, ws, scratch_bytes, s, mask,
                         mask_stride);
}

void launch_apply_mask(float *scores, int64_t nq, int64_t ld, int64_t nc, const uint8_t *mask, int64_t mask_stride,
                       const int64_t *row_map, int64_t col0, hipStream_t s)
{
    apply_mask(scores, nq, ld, nc, mask, mask_stride, row_map, col0, s);
}
void launch_apply_mask(int32_t *scores, int64_t nq, int64_t ld, int64_t nc, const uint8_t *mask, int64_t mask_stride,
                       const int64_t *row_map, int64_t col0, hipStream_t s)
{
    apply_mask(scores, nq, ld, nc, mask, mask_stride, row_map, col0, s);
}
void launch_drop_worst_keys_f32(unsigned long long *keys, int64_t n, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(drop_worst_keys_kernel<float>, dim3(blocks_for(n)), dim3(256), 0, s, keys, n);
    }
}
void launch_drop_worst_keys_i32(unsigned long long *keys, int64_t n, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(drop_worst_keys_kernel<int32_t>, dim3(blocks_for(n)), dim3(256), 0, s, keys, n);
    }
}

int stream_select_bf16x3(const uint16_t *Qs, int64_t nq, const uint16_t *Bs, int64_t nb, int d3, const float *qn,
                         const float *bn, int metric, int ncand, unsigned long long *running,
                         StreamSelectWorkspace<float> &ws, int64_t scratch_bytes, hipStream_t s)
{
    // the ring kernel needs whole K-steps and at least 2048 base rows in every launch; a plan with a
    // narrower chunk (a small scratch, a short remainder) answers -1 as well
    if (d3 % 32 != 0 || nb < 2048 || reinterpret_cast<uintptr_t>(Qs) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(Bs) % 16 != 0) {
        return -1;
    }
    return stream_select(Bf16Ops{qn, bn, metric}, Qs, nq, Bs, nb, d3, ncand, running, ws, scratch_bytes, s);
}

// ---- bound by sample, proof afterwards --------------------------------------------------------------
// The plan for large query x base products that need only a few keys per row (the IVFPQ coarse stage):
// no score is ever written to memory except the few a row admits.
//   1. a group-minima launch over a seed stretch (the first `seed` base rows) leaves, per row, the
//      smallest score of each group of 32 seed rows: G = seed / 32 values;
//   2. tau = the j-th smallest of them, an upper bound of the j-th smallest seed score.  j is chosen so
//      that tau lies at or above the row's r-th smallest score over the WHOLE base with overwhelming
//      probability (r = the rank the caller's proof needs): the seed holds m = r seed / nb of the true
//      best r on average (hypergeometric, variance < m), and j = m + 4.5 sqrt(m) + 3;
//   3. one record-mode launch over the whole base appends every run of four scores with a score <= tau;
//   4. a fold turns the records into the result and PROVES it per row (launch_fold_records: at least
//      ncand scores <= tau; launch_fold_refine_boundary: tau above the decision band of rank nout).
//      Rows without proof (tau too low after all, or records dropped) are appended to `flag` for the
//      caller's exact plan.
// About nb (1 - (1 - j / G)^(1/32)) scores per row are admitted instead of nb written and read again.
// Base rows are assumed to come in no particular order (k-means centroids do); an order that makes the
// seed unrepresentative only costs proofs, never correctness.  No host synchronisation.
// Returns the number of score launches, or -1 when the plan does not apply (nothing has been queued).
int stream_select_bf16x3_sampled(const uint16_t *Qs, int64_t nq_total, const uint16_t *Bs, int64_t nb_total, int d3,
                                 const float *qn, const float *bn, int metric, int ncand, unsigned long long *running,
                                 StreamSelectWorkspace<float> &ws, int64_t scratch_bytes, int *flag,
                                 const BoundaryRefine *refine, hipStream_t s, const ResidentCoarse *resident)
{
    if (resident && !resident_coarse_serves(d3)) {
        resident = nullptr;
    }
    if (!flag || d3 % 32 != 0 || nb_total % 4 != 0 || ncand > kFoldMaxK || reinterpret_cast<uintptr_t>(Qs) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(Bs) % 16 != 0) {
        return -1;
    }
    const int64_t seed = round_up(std::max<int64_t>(2048, 16 * (int64_t)ncand), 256);
    if (nb_total < 4 * seed || nq_total * nb_total < ((int64_t)16 << 20)) {
        return -1;   // short bases and small products: one materialised pass is cheaper
    }
    const int G = (int)(seed / 32);
    // the rank tau has to reach: the whole candidate list, or rank nout plus room for its decision band
    const int r = refine ? std::min(ncand, refine->nout + 8 + refine->nout / 16) : ncand;
    const double m = (double)r * (double)seed / (double)nb_total;
    const int j = (int)std::ceil(m + 4.5 * std::sqrt(m) + 3.0);
    if (4 * j > 3 * G) {
        return -1;   // the seed is too small a sample for this rank
    }
    // expected scores <= tau per row: a group's minimum is <= tau with probability j / G
    const double admitted = (1.0 - std::pow(1.0 - (double)j / G, 1.0 / 32.0)) * (double)nb_total;
    // How many a row may admit: tau is the j-th of G order statistics, so the share of groups below it scatters by
    // about 1 / sqrt(j) of its mean -- twice the expectation is five deviations at j = 27 (a search for 64 lists) and
    // fewer than three at j = 7 (an assignment among 65536 centroids: 0.6 % of the rows overflowed their records
    // and were redone exactly), so small j get more room.
    const double slack = std::max(2.0, 1.0 + 6.0 / std::sqrt((double)j));
    if (r + slack * admitted > 2048.0) {
        return -1;   // more than a fold holds
    }
    const int capk = (int)std::ceil(r + slack * admitted);                     // scores <= tau a row may have
    const int cap = std::max(256, pow2_ceil((int)std::ceil(slack * admitted)));   // records per row
    int64_t qb = std::min<int64_t>(round_up(nq_total, 128), 16384);
    if (scratch_bytes / ((int64_t)cap * 32) < qb) {   // the records of a query block stay inside the scratch budget
        qb = scratch_bytes / ((int64_t)cap * 32) / 128 * 128;
        if (qb < 128) {
            return -1;
        }
    }
    ws.scores.resize((size_t)qb * G);
    ws.tau.resize((size_t)nq_total);
    if (resident) {
        ws.thr.resize((size_t)nq_total);   // the record launch's per-query test values
    }
    const bool fresh_cnt = ws.cnt.size() < (size_t)nq_total + 1;
    ws.cnt.resize((size_t)nq_total + 1);
    ws.filter.resize((size_t)qb * cap * 4);   // 32-byte records
    if (fresh_cnt || !ws.cnt_zero) {
        IXA_HIP(hipMemsetAsync(ws.cnt.data(), 0, ws.cnt.bytes(), s));   // the folds leave the counters at zero
    }
    ws.cnt_zero = false;   // until every fold below has been queued
    int launches = 0;
    for (int64_t q0 = 0; q0 < nq_total; q0 += qb) {
        const int64_t nq = std::min(qb, nq_total - q0);
        bool ok = resident ? launch_resident_bf16_minima(Qs + q0 * d3, nq, resident->Bt, seed, d3, qn + q0,
                                                         resident->cn_padded, metric, ws.scores.data(), G, s)
                           : launch_score_ring_bf16_minima(Qs + q0 * d3, nq, Bs, seed, d3, qn + q0, bn, metric,
                                                           ws.scores.data(), G, s);
        IXA_REQUIRE(ok, kErrInner, "bf16 score kernel rejected a shape it had accepted");
        const RecordTest rt{qn + q0, resident ? resident->cmax : 0.f, metric, resident ? ws.thr.data() + q0 : nullptr};
        launch_tau_from_minima(ws.scores.data(), G, j, nq, ws.tau.data() + q0, s, resident ? &rt : nullptr);
        ScoreFilter<float> flt{ws.tau.data() + q0, nullptr, ws.cnt.data() + q0, ws.filter.data(), cap, 0};
        ok = resident ? launch_resident_bf16_records(Qs + q0 * d3, nq, resident->Bt, nb_total, d3, qn + q0,
                                                     resident->cn_padded, metric, ws.thr.data() + q0, flt, s)
                      : launch_score_ring_bf16_records(Qs + q0 * d3, nq, Bs, nb_total, d3, qn + q0, bn, metric, flt, s);
        IXA_REQUIRE(ok, kErrInner, "bf16 score kernel rejected a shape it had accepted");
        // the resident-query launch records dot products; the folds form the scores
        const RawRecords raw{qn + q0, bn, metric};
        if (refine) {
            // only the exact best-nout SET is wanted: no sorted list in between
            launch_fold_refine_boundary(refine->Q + q0 * refine->d, nq, refine->C, refine->d, qn + q0, bn, metric, flt,
                                        capk, refine->nout, refine->cmax, refine->err_scale, refine->round_scale,
                                        refine->out_ids + q0 * refine->nout, flag, q0, s, resident != nullptr);
        } else {
            launch_fold_records(running + q0 * ncand, ncand, flt, nq, flag, q0, s, resident ? &raw : nullptr);
        }
        launches += 2;
    }
    ws.cnt_zero = true;
    return launches;
}

int stream_select_i8(const int8_t *Q, int64_t nq, const int8_t *B, int64_t nb, int d, const int32_t *qn,
                     const int32_t *bn, int ncand, unsigned long long *running, StreamSelectWorkspace<int32_t> &ws,
                     int64_t scratch_bytes, hipStream_t s, const uint8_t *mask, int64_t mask_stride)
{
    return stream_select(I8Ops{qn, bn}, Q, nq, B, nb, d, ncand, running, ws, scratch_bytes, s, mask, mask_stride);
}

void launch_keys_to_idx(const unsigned long long *keys, int64_t n, int32_t *idx, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(keys_to_idx_kernel, dim3(blocks_for(n)), dim3(256), 0, s, keys, n, idx);
    }
}

}  // namespace ixa
