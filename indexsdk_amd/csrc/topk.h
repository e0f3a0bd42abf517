// Device-side top-k building blocks for 64-wide wavefronts (gfx950).
//
// Every candidate is a 64-bit key  (ordered(score) << 32) | index  where "score" is the quantity
// to MINIMISE (the L2 distance, or the negated inner product) and index is a 32-bit position
// (arena slot / centroid id / base row).  Smaller key == better candidate; exact score ties
// resolve to the smaller index.  A key of all ones is the empty slot.
//
// WavePool: each wavefront keeps a private pool of candidates in LDS.  A candidate enters only
// if its score is <= the wave's current bound; when the pool fills, the wave sorts it (bitonic,
// in LDS, wave-synchronous: no workgroup barrier), keeps the best k and tightens the bound to
// the k-th score.  Waves of a workgroup publish their bounds so that each can adopt the minimum.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace ixa {

using key_t = unsigned long long;
constexpr key_t kEmptyKey = ~0ull;
constexpr int kWave = 64;

__device__ __forceinline__ uint32_t ordered_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}

__device__ __forceinline__ float unordered_bits(uint32_t o)
{
    uint32_t u = o ^ ((o >> 31) ? 0x80000000u : 0xffffffffu);
    return __uint_as_float(u);
}

// int32 scores (exact integer distances) order by flipping the sign bit.
__device__ __forceinline__ uint32_t ordered_bits(int32_t v) { return (uint32_t)v ^ 0x80000000u; }

template <typename S>
struct ScoreOps;
template <>
struct ScoreOps<float> {
    static __device__ __forceinline__ float from_ordered(uint32_t o) { return unordered_bits(o); }
    static __device__ __forceinline__ float worst() { return __builtin_inff(); }
};
template <>
struct ScoreOps<int32_t> {
    static __device__ __forceinline__ int32_t from_ordered(uint32_t o) { return (int32_t)(o ^ 0x80000000u); }
    static __device__ __forceinline__ int32_t worst() { return 0x7fffffff; }
};

__device__ __forceinline__ float wave_uniform(float v)
{
    return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v)));
}
__device__ __forceinline__ int32_t wave_uniform(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }

template <typename S>
__device__ __forceinline__ key_t make_key(S score, uint32_t idx)
{
    return ((key_t)ordered_bits(score) << 32) | idx;
}
__device__ __forceinline__ float key_score(key_t k) { return unordered_bits((uint32_t)(k >> 32)); }
template <typename S>
__device__ __forceinline__ S key_score_as(key_t k)
{
    return ScoreOps<S>::from_ordered((uint32_t)(k >> 32));
}
__device__ __forceinline__ uint32_t key_index(key_t k) { return (uint32_t)k; }

// Orders LDS traffic of ONE wavefront (its lanes exchange data through LDS without s_barrier).
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

// Bitonic sort (ascending) of n = power-of-two keys in LDS by the lanes of one wavefront.
__device__ inline void wave_bitonic_sort(key_t *buf, int n, int lane)
{
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            wave_lds_fence();
            for (int t = lane; t < (n >> 1); t += kWave) {
                int i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                int j = i + stride;
                bool up = (i & size) == 0;
                key_t a = buf[i], b = buf[j];
                if ((a > b) == up) {
                    buf[i] = b;
                    buf[j] = a;
                }
            }
        }
    }
    wave_lds_fence();
}

// Same sort, executed by a whole workgroup with barriers (used for the final merge).
__device__ inline void block_bitonic_sort(key_t *buf, int n, int tid, int nthreads)
{
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int t = tid; t < (n >> 1); t += nthreads) {
                int i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                int j = i + stride;
                bool up = (i & size) == 0;
                key_t a = buf[i], b = buf[j];
                if ((a > b) == up) {
                    buf[i] = b;
                    buf[j] = a;
                }
            }
        }
    }
    __syncthreads();
}

template <typename S = float>
struct WavePool {
    key_t *buf;   // LDS, cap entries, private to this wave
    int cap;      // power of two, >= k + 2 * kWave
    int k;
    int count;    // wave-uniform
    S bound;      // wave-uniform: a candidate enters iff score <= bound

    __device__ __forceinline__ void init(key_t *b, int cap_, int k_)
    {
        buf = b;
        cap = cap_;
        k = k_;
        count = 0;
        bound = ScoreOps<S>::worst();
    }

    // Sort, keep the best k, tighten the bound.  All lanes of the wave must call it.
    __device__ inline void compact(int lane)
    {
        for (int i = count + lane; i < cap; i += kWave) {
            buf[i] = kEmptyKey;
        }
        wave_bitonic_sort(buf, cap, lane);
        if (count > k) {
            count = k;
        }
        if (count == k) {
            S b = wave_uniform(key_score_as<S>(buf[k - 1]));
            bound = b < bound ? b : bound;
        }
    }

    // All lanes call; lanes with pass == false contribute nothing.  Returns true when the
    // pool was compacted (the bound may have tightened).
    __device__ __forceinline__ bool push(bool pass, S score, uint32_t idx, int lane)
    {
        unsigned long long mask = __ballot(pass);
        if (mask == 0) {
            return false;
        }
        int pre = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        if (pass) {
            buf[count + pre] = make_key(score, idx);
        }
        count += __popcll(mask);
        if (count > cap - kWave) {
            compact(lane);
            return true;
        }
        return false;
    }
};

inline int wave_pool_capacity(int k)
{
    int cap = 256;
    while (cap < k + 2 * kWave) {
        cap <<= 1;
    }
    return cap;
}

}  // namespace ixa
