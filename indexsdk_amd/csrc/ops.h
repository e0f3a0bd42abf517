// Stage operators of the IVFPQ search path, one launch each (see ops.hip).
#pragma once
#include "common.h"

namespace ixa {

// dist[batch][n] and, when mins != nullptr, mins[batch][ceil(n / 64) * 2] = (minimum, position in the
// burst as uint32 bits) of every burst of 64 codes.
void op_distance_flat_l2_mins_fp32(const float *queries, int64_t batch, const float *codes, int64_t n, int d,
                                   const float *codes_sqr_sum, float *dist, float *mins, hipStream_t s);

// lut[batch][M][256] from queries[batch][d] and codebook[M][256][d / M].
void op_ivfpq_subspace_distance(const float *queries, int64_t batch, int d, const float *codebook, int M, int metric,
                                float *lut, hipStream_t s);

// The k smallest of every row of dists[batch][ld] (first n columns), ascending, ties to the lower
// column; rows shorter than k are padded with (FLT_MAX, -1).
void op_topk_flat_fp32(const float *dists, int64_t batch, int64_t n, int64_t ld, int k, float *out_dist,
                       int64_t *out_label, hipStream_t s);

}  // namespace ixa
