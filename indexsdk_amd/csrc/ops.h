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

// The fused scan + top-k with the reference's operands: lut[batch][M][256], code blocks at code_base +
// code_offset[batch][nblk] (bytes) with code_size[batch][nblk] valid codes each (row-major, M bytes per code),
// labels at label_base[label_offset[batch][nblk] + position]; out: the k best per query, best first, padded with
// (FLT_MAX or -FLT_MAX, -1).  k <= 384, nblk <= 2048, blocks of at most 262144 codes.
void op_ivfpq_search_distance_topk(const float *lut, int64_t batch, int M, const uint8_t *code_base,
                                   const int64_t *code_offset, const int64_t *code_size, int nblk, int k,
                                   const int64_t *label_base, const int64_t *label_offset, int metric, float *out_val,
                                   int64_t *out_lab, hipStream_t s);

// Merges in_labels / in_values [T][batch][K] (best first per list, label -1 = padding) into the k best per query.
void op_topk_ivfpq_l3(const int64_t *in_labels, const float *in_values, int T, int64_t batch, int K, int k, int asc,
                      float *out_values, int64_t *out_labels, hipStream_t s);

}  // namespace ixa
