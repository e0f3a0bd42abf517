// Host launchers of the stage-1 kernels (score tiles, row selection, exact refine).
#pragma once
#include "common.h"

namespace ixa {

// out[i] = |x_i|^2, accumulated left to right in fp32.
void launch_sqnorm_rows(const float *x, int64_t n, int d, float *out, hipStream_t s);

// Filtered epilogue of the score kernels: instead of storing the scores, every score <= tau[row]
// is appended as a key (ordered score << 32 | col_base + col) to cand[row * cap + cnt[row]++].
// cnt may run past cap (the excess is dropped); the merge step reports that as an overflow.
template <typename S>
struct ScoreFilter {
    const S *tau;              // [nq] admission bound per row
    const S *thr;              // [nq] tau - |q|^2 (exact integer scores only; may be null)
    int32_t *cnt;              // [nq] number of appended keys
    unsigned long long *cand;  // [nq][cap]
    int cap;
    int64_t col_base;
};

// out[row * ldo + col] = score(Q[row], C[col]) for row < nq, col < nc (fp32 MFMA).
void launch_score_tiles(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                        const float *cn, int metric, float *out, int64_t ldo, hipStream_t s);

void launch_score_tiles_filtered(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                                 const float *cn, int metric, ScoreFilter<float> flt, hipStream_t s);

// Merges the filtered candidates of every row into its running best-k keys (sorted, kEmptyKey
// padded), sets tau[row] to the k-th score (or leaves it when fewer than k keys exist), resets
// cnt[row] and raises *overflow when a row had appended more than cap keys.
void launch_merge_candidates(unsigned long long *running, int k, ScoreFilter<float> flt, float *tau, int64_t nq,
                             int *overflow, hipStream_t s);
// thr (may be null): thr[row] = min(new tau, max_bound) - qn[row] is written along with tau[row], the threshold form the
// int8 score kernels filter by
void launch_merge_candidates_i32(unsigned long long *running, int k, ScoreFilter<int32_t> flt, int32_t *tau,
                                 int64_t nq, int *overflow, hipStream_t s, int32_t *thr = nullptr,
                                 const int32_t *qn = nullptr, int32_t max_bound = 0);

// Persistent ring kernels (score_ring.hip): same results as the tile kernels, at a much higher
// matrix-core rate.  Return false when the shape does not qualify (d not a multiple of one K-step,
// fewer than 1024 base rows, unaligned operands); nothing has been launched then.
bool launch_score_ring_f32(const float *Q, int64_t nq, const float *B, int64_t nb, int d, const float *qn,
                           const float *bn, int metric, float *out, int64_t ldo, bool filter, ScoreFilter<float> flt,
                           hipStream_t s);

bool launch_score_ring_bf16(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                            const float *bn, int metric, float *out, int64_t ldo, bool filter, ScoreFilter<float> flt,
                            hipStream_t s);

// The same two launches with the query tile resident in LDS and the split centroids read from matrix-core order
// (coarse_resident.hip): Bt = the base-side split rows tiled as flat_i8.h describes (rows of 2 d3 bytes, whole tiles of
// 256 rows, zero rows behind the last), cn_padded = |c|^2 per row (zeros for inner product) padded to whole tiles with
// +inf.  The records hold DOT PRODUCTS, not scores: the folds below take them with raw = true.  test: the per-row
// values of record_test_value (launch_tau_from_minima writes them).  Return false (nothing launched) for split rows
// they have no instance for.
bool resident_coarse_serves(int d3);
bool launch_resident_bf16_minima(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, int64_t nb, int d3, const float *qn,
                                 const float *cn_padded, int metric, float *out, int64_t ldo, hipStream_t s);
bool launch_resident_bf16_records(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, int64_t nb, int d3, const float *qn,
                                  const float *cn_padded, int metric, const float *test, ScoreFilter<float> flt,
                                  hipStream_t s);

// Record mode of the bf16 ring kernel: nothing is stored; every run of four consecutive base rows (first
// row a multiple of four) whose smallest score is at or below flt.tau[row] is appended to the row's
// record list: 32 bytes {four fp32 scores, uint32 col_base + first base row, unused} at
// (unsigned char *)flt.cand + (row * flt.cap + i) * 32, i counted in flt.cnt[row] (which may run past
// flt.cap: the excess is dropped and the folds below treat such a row as unproven).  nb % 4 == 0.
bool launch_score_ring_bf16_records(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                                    const float *bn, int metric, ScoreFilter<float> flt, hipStream_t s);
// Group-minima mode: out[row * ldo + g] = the smallest score of the row among the 32 base rows of group g, for
// the 8 * ceil(nb / 256) groups of the base (+inf for a group past its end); each base row is in exactly one
// group.  Nothing else is written.  nb % 4 == 0.
bool launch_score_ring_bf16_minima(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                                   const float *bn, int metric, float *out, int64_t ldo, hipStream_t s);
// tau[row] = the rank-th smallest (1-based) of gm[row * G .. + G); G <= 512.
// With `test`, test->out[row] also receives the value the resident-query record launch compares against
// (record_test_value below), so that launch needs no kernel of its own in front of it.
//   A run is recorded when some u = g - |c|^2 / 2 of its four reaches the test value.
//   L2: score v = fl(fl(fl(|q|^2 + |c|^2) - g) - g) <= tau.  v differs from |q|^2 + |c|^2 - 2 g by at most three
//   roundings of numbers no larger than |q|^2 + |c|^2 + 2 |g| <= 2 (|q|^2 + |c|^2): 6 x 2^-24 (|q|^2 + |c|^2); u differs
//   from g - |c|^2 / 2 by one rounding, at most 2^-24 (|q|^2 + |c|^2).  So v <= tau implies
//   u >= (|q|^2 - tau) / 2 - 4 x 2^-24 (|q|^2 + |c|^2); the test value lies another factor of two below that, with
//   |c| <= cmax, and below its own rounding.
//   Inner product: v = -g <= tau  <=>  g >= -tau, and u = g exactly (the norms handed to the kernel are zero).
__host__ __device__ inline float record_test_value(float qn, float tau, float cmax, bool l2)
{
    if (l2) {
        const float mag = qn + cmax * cmax + (tau < 0.f ? -tau : tau);
        return 0.5f * (qn - tau) - 4.8e-7f * mag;   // 2^-21 = 4.77e-7
    }
    return -tau - 4.8e-7f * (tau < 0.f ? -tau : tau);
}
struct RecordTest {
    const float *qn;   // |q|^2 per row
    float cmax;        // largest centroid norm
    int metric;
    float *out;
};
void launch_tau_from_minima(const float *gm, int G, int rank, int64_t nq, float *tau, hipStream_t s,
                            const RecordTest *test = nullptr);

// Largest k of launch_fold_records.
constexpr int kFoldMaxK = 384;
// Turns the records of a launch over the WHOLE base into every row's best-k keys (running[nq][k], sorted,
// kEmptyKey padded; written only), resets cnt[row], and appends every row whose result is not PROVEN to be
// the k smallest keys of the base (fewer than k scores <= tau[row] on record, or records dropped) to
// flag[1 + flag[0]++] as row_base + row, marking it by kEmptyKey in its last key.
// raw (may be null): the records hold dot products (launch_resident_bf16_records); scores are formed from them with
// these row and column norms (cn 16-byte aligned; unused for inner product)
struct RawRecords {
    const float *qn, *cn;
    int metric;
};
void launch_fold_records(unsigned long long *running, int k, ScoreFilter<float> flt, int64_t nq, int *flag,
                         int64_t row_base, hipStream_t s, const RawRecords *raw = nullptr);
// launch_fold_records and launch_refine_boundary in one launch, without the sort in between: the exact best
// nout SET of every row; capk = scores <= tau a row may have on record (at most 2048); rows without proof
// are appended to flag.  Resets cnt[row].
void launch_fold_refine_boundary(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn,
                                 int metric, ScoreFilter<float> flt, int capk, int nout, float cmax, float err_scale,
                                 float round_scale, int32_t *out_ids, int *flag, int64_t row_base, hipStream_t s,
                                 bool raw = false);

// out[row] = [hi | hi | lo] (query side) or [hi | lo | hi] (base side) of x[row], each segment
// zero-padded from d to dp elements of bf16 (stored as uint16_t); out has n * 3 * dp elements.
void launch_split_bf16x3(const float *x, int64_t n, int d, int dp, bool base_side, uint16_t *out, hipStream_t s);
// launch_sqnorm_rows(x -> norms) and the query-side launch_split_bf16x3(x -> split) in one launch
void launch_sqnorm_and_split_bf16x3(const float *x, int64_t n, int d, int dp, float *norms, uint16_t *split, hipStream_t s);

// Sets *flag = 1 if some query's approximate candidate list (running[nq][ncand], ascending keys) is
// not provably a superset of its best nout centroids; see score_ring.hip.
void launch_verify_superset(const unsigned long long *running, int ncand, const float *exact_dist, int nout,
                            const float *qn, float cmax, float err_scale, float round_scale, int metric, int64_t nq,
                            int *flag,
                            hipStream_t s);

// Largest selection size of launch_select_rows*: the private pools of its wavefronts hold 4096 keys.
constexpr int kSelectMaxK = 3072;

// Best `ksel` columns of every row of a score matrix.  out_idx (may be null) receives the column
// indices (+ col_base), best first.  running (may be null) is a [nrows][ksel] array of keys
// (ordered score << 32) | (col_base + column): its content takes part in the selection and is
// replaced by the result, so calling this over successive column chunks keeps a streaming top-k.
// Before the first chunk fill it with 0xff bytes, or pass fresh = true for that chunk (`running` is then
// only written).
void launch_select_rows(const float *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                        int64_t col_base, unsigned long long *running, hipStream_t s, bool fresh = false);
void launch_select_rows_i32(const int32_t *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                            int64_t col_base, unsigned long long *running, hipStream_t s, bool fresh = false);

// Exact best-nout SET from approximately scored, sorted candidates (see refine_boundary_kernel):
// re-evaluates only the candidates within 2 * err of the rank-nout score; a query whose list
// cannot be proven to contain every winner is appended to flag[1 + flag[0]++] (flag: 1 + nq ints); complete = the
// candidates are ALL base rows, so nothing is left to prove.  out_ids: [nq][nout], unordered.
void launch_refine_boundary(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn,
                            int metric, const unsigned long long *running, int ncand, int nout, float cmax,
                            float err_scale, float round_scale, int32_t *out_ids, int *flag, bool complete,
                            hipStream_t s);

// Canonical scores of all nc centroids for every row (one lane per score; the exact plan of last resort).
void launch_canonical_scores(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                             const float *cn, int metric, float *out, int64_t ldo, hipStream_t s);
// dist[n][k] = public distances of the columns idx[n][k] of a score matrix (-1 -> +-FLT_MAX).
void launch_gather_scores(const float *scores, int64_t ld, const int32_t *idx, int64_t n, int k, int metric, float *dist,
                          hipStream_t s);

// Canonical re-evaluation of cand[nq][ncand] (-1 = absent) and selection of the best nout.  Rows of
// the outputs are out_stride (>= nout) wide; columns past nout are padded with (-1, +-FLT_MAX).
void launch_refine(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn, int metric,
                   const int32_t *cand, int ncand, int nout, int out_stride, int32_t *out_ids, float *out_dist,
                   hipStream_t s);

}  // namespace ixa
