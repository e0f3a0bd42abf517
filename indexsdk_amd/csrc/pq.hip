// PQ encode on the GPU, bit-exact to the reference's host encoder
// (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:879-921: encodeSingleVectorPQ /
// findCentroidInSubQuantizer / calDistance): the RAW vector is encoded (by_residual = false),
// distance = sum (a-b)^2 accumulated left to right in fp32 without FMA, strict '<' so the first
// minimum wins.  This is plain VALU work: the arithmetic order is the contract, so it is not
// reshaped into a GEMM.
#include "pq.h"

namespace ixa {

// One workgroup finds the codes of 256 vectors for ONE sub-quantizer (blockIdx.y): its 256 x dsub codeword
// slab is staged in LDS and every lane walks all 256 codewords for its own vector (all lanes read the same
// LDS address per step: a broadcast, no bank conflicts).  A small batch still fills the GPU this way: the
// walk is a serial chain per lane, and 10000 vectors x 32 sub-quantizers are 1280 workgroups instead of 40.
template <int DSUB>
__global__ __launch_bounds__(256) void pq_encode_kernel(const float *__restrict__ x, int64_t n, int d, int M,
                                                        const float *__restrict__ codebook,
                                                        uint8_t *__restrict__ codes)
{
    __shared__ float cb[256 * DSUB];
    const int tid = threadIdx.x;
    const int m = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * 256 + tid;
    const float *src = codebook + (int64_t)m * 256 * DSUB;
    for (int e = tid; e < 256 * DSUB; e += 256) {
        cb[e] = src[e];
    }
    __syncthreads();
    if (i < n) {
        float sub[DSUB];
#pragma unroll
        for (int t = 0; t < DSUB; t++) {
            sub[t] = x[i * d + (int64_t)m * DSUB + t];
        }
        float best = 3.402823466e+38f;
        int arg = 0;
        for (int k = 0; k < 256; k++) {
            float dist = 0.f;
#pragma unroll
            for (int t = 0; t < DSUB; t++) {
                float diff = __fsub_rn(sub[t], cb[k * DSUB + t]);
                dist = __fadd_rn(dist, __fmul_rn(diff, diff));
            }
            if (dist < best) {
                best = dist;
                arg = k;
            }
        }
        codes[i * M + m] = (uint8_t)arg;
    }
}

// Any dsub: the sub-vector is re-read from global memory (cached) instead of living in registers.
__global__ __launch_bounds__(256) void pq_encode_generic_kernel(const float *__restrict__ x, int64_t n, int d, int M,
                                                                int dsub, const float *__restrict__ codebook,
                                                                uint8_t *__restrict__ codes)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (i >= n) {
        return;
    }
    const float *sub = x + i * d + (int64_t)m * dsub;
    const float *cb = codebook + (int64_t)m * 256 * dsub;
    float best = 3.402823466e+38f;
    int arg = 0;
    for (int k = 0; k < 256; k++) {
        float dist = 0.f;
        for (int t = 0; t < dsub; t++) {
            float diff = __fsub_rn(sub[t], cb[k * dsub + t]);
            dist = __fadd_rn(dist, __fmul_rn(diff, diff));
        }
        if (dist < best) {
            best = dist;
            arg = k;
        }
    }
    codes[i * M + m] = (uint8_t)arg;
}

void launch_pq_encode(const float *x, int64_t n, int d, int M, const float *codebook, uint8_t *codes, hipStream_t s)
{
    if (n == 0) {
        return;
    }
    const int dsub = d / M;
    dim3 grid((unsigned)((n + 255) / 256), (unsigned)M), block(256);
#define IXA_ENC(D)                                                                                             \
    case D:                                                                                                    \
        hipLaunchKernelGGL(pq_encode_kernel<D>, grid, block, 0, s, x, n, d, M, codebook, codes);              \
        break;
    switch (dsub) {
        IXA_ENC(1)
        IXA_ENC(2)
        IXA_ENC(3)
        IXA_ENC(4)
        IXA_ENC(6)
        IXA_ENC(8)
        IXA_ENC(12)
        IXA_ENC(16)
        IXA_ENC(24)
        IXA_ENC(32)
        default:
            hipLaunchKernelGGL(pq_encode_generic_kernel, grid, block, 0, s, x, n, d, M, dsub, codebook, codes);
    }
#undef IXA_ENC
}

}  // namespace ixa
