// Host launchers of the stage-1 kernels (score tiles, row selection, exact refine).
#pragma once
#include "common.h"

namespace ixa {

// out[i] = |x_i|^2, accumulated left to right in fp32.
void launch_sqnorm_rows(const float *x, int64_t n, int d, float *out, hipStream_t s);

// out[row * ldo + col] = score(Q[row], C[col]) for row < nq, col < nc (fp32 MFMA).
void launch_score_tiles(const float *Q, int64_t nq, const float *C, int64_t nc, int d, const float *qn,
                        const float *cn, int metric, float *out, int64_t ldo, hipStream_t s);

// Best `ksel` columns of every row of a score matrix; out_idx and/or out_keys may be null.
// out_keys carry (ordered score << 32) | (col_base + column).
void launch_select_rows(const float *scores, int64_t nrows, int64_t ld, int64_t nc, int ksel, int32_t *out_idx,
                        int64_t col_base, unsigned long long *out_keys, hipStream_t s);

// Canonical re-evaluation of cand[nq][ncand] (-1 = absent) and selection of the best nout.
void launch_refine(const float *Q, int64_t nq, const float *C, int d, const float *qn, const float *cn, int metric,
                   const int32_t *cand, int ncand, int nout, int32_t *out_ids, float *out_dist, hipStream_t s);

}  // namespace ixa
