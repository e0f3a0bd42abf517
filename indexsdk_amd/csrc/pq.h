// Host launchers of the product-quantizer kernels (codeword norms, exact encode).
#pragma once
#include "common.h"

namespace ixa {

// codes[i][m] = first argmin_k sum_t (x[i][m*dsub+t] - codebook[m][k][t])^2, fp32, left to right.
void launch_pq_encode(const float *x, int64_t n, int d, int M, const float *codebook, uint8_t *codes, hipStream_t s);

}  // namespace ixa
