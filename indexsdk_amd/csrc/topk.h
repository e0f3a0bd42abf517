// Device-side top-k building blocks for 64-wide wavefronts (gfx950).
//
// Every candidate is a 64-bit key  (ordered(score) << 32) | index  where "score" is the quantity
// to MINIMISE (the L2 distance, the negated inner product, or an exact int32 distance) and index
// is a 32-bit position (arena slot / centroid id / base row).  Smaller key == better candidate;
// exact score ties resolve to the smaller index.  A key of all ones is the empty slot.
//
// WavePool: each wavefront keeps a private, UNSORTED pool of candidates in LDS.  A candidate
// enters only if its score is <= the wave's current bound.  When the pool fills, the wave finds
// (by a bitwise search over the top 20 bits of the ordered scores, one ballot per key and bit) the
// smallest score bucket that still holds k candidates, drops everything above it and tightens its
// bound to the top of that bucket -- no sorting, no workgroup barrier.  The same search at rank
// ceil(k / W) gives a value every wave publishes; the maximum of the W published values has at
// least k candidates below it across the workgroup, so every wave may adopt it as its bound.
// Sorting happens once, at the end, on the few survivors of all pools.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace ixa {

using key_t = unsigned long long;
constexpr key_t kEmptyKey = ~0ull;
constexpr int kWave = 64;
constexpr int kSelectBits = 20;  // resolution of the bucket search (sign + exponent + 11 mantissa bits)

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
    // largest score of the bucket with the given ordered prefix (never NaN)
    static __device__ __forceinline__ float bucket_top(uint32_t o)
    {
        float v = unordered_bits(o);
        return v == v ? v : __builtin_inff();
    }
};
template <>
struct ScoreOps<int32_t> {
    static __device__ __forceinline__ int32_t from_ordered(uint32_t o) { return (int32_t)(o ^ 0x80000000u); }
    static __device__ __forceinline__ int32_t worst() { return 0x7fffffff; }
    static __device__ __forceinline__ int32_t bucket_top(uint32_t o) { return (int32_t)(o ^ 0x80000000u); }
};

__device__ __forceinline__ float wave_uniform(float v)
{
    return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(v)));
}
__device__ __forceinline__ int32_t wave_uniform(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ key_t wave_uniform_key(key_t v)
{
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return ((key_t)hi << 32) | lo;
}

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

// Same sort, executed by a whole workgroup with barriers.
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
    key_t *buf;   // LDS, cap entries, private to this wave, unsorted
    int cap;      // power of two, >= k + 2 * kWave
    int k;
    int count;    // wave-uniform
    S bound;      // wave-uniform: a candidate enters iff score <= bound
    // Wave-uniform; set once so many candidates TIE at the k-th score that a bound on scores alone keeps
    // admitting them (coarse quantizers give whole lists one code): from then on a candidate must also be
    // below this key, the k-th smallest (score, index) seen, so ties are decided by index as in the result.
    key_t bound_key;

    __device__ __forceinline__ void init(key_t *b, int cap_, int k_)
    {
        buf = b;
        cap = cap_;
        k = k_;
        count = 0;
        bound = ScoreOps<S>::worst();
        bound_key = kEmptyKey;
    }

    // Smallest kSelectBits-bit prefix P such that at least `rank` pool entries have a score prefix
    // <= P.  Requires 1 <= rank <= count.  Wave-uniform result.
    __device__ inline uint32_t select_prefix(int rank, int lane) const
    {
        constexpr int SH = 32 - kSelectBits;
        uint32_t P = 0;
        if (count <= 4 * kWave) {
            // common case: up to four prefixes per lane live in registers
            uint32_t pre[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int i = j * kWave + lane;
                pre[j] = i < count ? (uint32_t)(buf[i] >> (32 + SH)) : 0xffffffffu;
            }
            for (int b = kSelectBits - 1; b >= 0; b--) {
                const uint32_t c = P | ((1u << b) - 1u);
                int cnt = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    cnt += __popcll(__ballot(pre[j] <= c));
                }
                if (cnt < rank) {
                    P |= 1u << b;
                }
            }
            return P;
        }
        for (int b = kSelectBits - 1; b >= 0; b--) {
            const uint32_t c = P | ((1u << b) - 1u);
            int cnt = 0;
            for (int i0 = 0; i0 < count; i0 += kWave) {
                const int i = i0 + lane;
                const uint32_t pre = i < count ? (uint32_t)(buf[i] >> (32 + SH)) : 0xffffffffu;
                cnt += __popcll(__ballot(pre <= c));
            }
            if (cnt < rank) {
                P |= 1u << b;
            }
        }
        return P;
    }

    // Keeps the entries whose score is <= limit (in place, order preserved).
    __device__ inline void keep_below(S limit, int lane)
    {
        int kept = 0;
        for (int i0 = 0; i0 < count; i0 += kWave) {
            const int i = i0 + lane;
            key_t kk = i < count ? buf[i] : kEmptyKey;
            const bool keep = i < count && key_score_as<S>(kk) <= limit;
            const unsigned long long mask = __ballot(keep);
            const int pre =
                __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
            wave_lds_fence();  // all reads of this chunk are done before anything is overwritten
            if (keep) {
                buf[kept + pre] = kk;  // kept + pre <= i: never ahead of the read frontier
            }
            kept += __popcll(mask);
        }
        wave_lds_fence();
        count = kept;
    }

    // Drops what cannot be among the k best and tightens the bound.  `share` (may be null) is
    // this wave's slot for the value at rank share_rank.  All lanes of the wave must call it.
    __device__ inline void compact(int lane, S *share, int share_rank)
    {
        constexpr int SH = 32 - kSelectBits;
        wave_lds_fence();
        if (share != nullptr && count >= share_rank) {
            const uint32_t Ps = select_prefix(share_rank, lane);
            const S top = ScoreOps<S>::bucket_top((Ps << SH) | ((1u << SH) - 1u));
            if (lane == 0 && top < *share) {
                *share = top;
            }
        }
        if (count < k) {
            return;
        }
        const uint32_t P = select_prefix(k, lane);
        const S top = ScoreOps<S>::bucket_top((P << SH) | ((1u << SH) - 1u));
        bound = top < bound ? top : bound;
        keep_below(bound, lane);
        if (count > cap - 2 * kWave) {
            // degenerate score distribution (one bucket holds almost everything): exact path
            for (int i = count + lane; i < cap; i += kWave) {
                buf[i] = kEmptyKey;
            }
            wave_bitonic_sort(buf, cap, lane);
            count = k;
            const key_t kth = wave_uniform_key(buf[k - 1]);
            const S b = key_score_as<S>(kth);
            bound = b < bound ? b : bound;
            bound_key = kth;   // keys are distinct: a later key that belongs to the k best is below this one
        }
    }

    // End of the stream: prune with the final bound so that the workgroup merge sees few keys.
    __device__ inline void finish(int lane)
    {
        if (count >= k) {
            compact(lane, nullptr, 0);
        } else {
            wave_lds_fence();
            keep_below(bound, lane);
        }
    }

    // All lanes call; lanes with pass == false contribute nothing.  Returns true when the
    // pool was compacted (the bound may have tightened).
    __device__ __forceinline__ bool push(bool pass, S score, uint32_t idx, int lane, S *share, int share_rank)
    {
        unsigned long long mask = __ballot(pass);
        if (mask == 0) {
            return false;
        }
        if (bound_key != kEmptyKey) {
            pass = pass && make_key(score, idx) < bound_key;
            mask = __ballot(pass);
            if (mask == 0) {
                return false;
            }
        }
        int pre = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        if (pass) {
            buf[count + pre] = make_key(score, idx);
        }
        count += __popcll(mask);
        if (count > cap - kWave) {
            compact(lane, share, share_rank);
            return true;
        }
        return false;
    }
};

// Workgroup epilogue: gathers the W pools (wave w owns pools[w*cap .. w*cap + counts[w])) to the
// front of the pool region, appends `extra_n` further keys (may be 0), sorts ascending and
// returns the number of valid keys; afterwards pools[0..result) is sorted.  The region must hold
// pow2_ceil(W*cap + extra_n) keys.  Called by all threads of the workgroup.
template <int W>
__device__ inline int block_merge_pools(key_t *pools, int cap, const int *counts, const key_t *extra, int extra_n,
                                        int tid)
{
    constexpr int NT = W * kWave;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < W; w++) {
        const int c = counts[w];
        if (w < wave) {
            before += c;
        }
        total += c;
    }
    // waves move their block to the left one after the other: the destination of wave w ends
    // where its own source begins at the latest, and never reaches into a block not yet moved
    for (int w = 1; w < W; w++) {
        if (wave == w) {
            const int c = counts[w];
            const key_t *src = pools + w * cap;
            for (int i0 = 0; i0 < c; i0 += kWave) {
                const int i = i0 + lane;
                key_t kk = i < c ? src[i] : kEmptyKey;
                wave_lds_fence();
                if (i < c) {
                    pools[before + i] = kk;
                }
            }
        }
        __syncthreads();
    }
    for (int i = tid; i < extra_n; i += NT) {
        pools[total + i] = extra[i];
    }
    total += extra_n;
    int n = 2;
    while (n < total) {
        n <<= 1;
    }
    for (int i = total + tid; i < n; i += NT) {
        pools[i] = kEmptyKey;
    }
    block_bitonic_sort(pools, n, tid, NT);
    return total;
}

// BlockPool: ONE unsorted candidate pool shared by the W wavefronts of a workgroup, for k too large
// for W private pools.  A wave reserves room with one LDS atomic per push.  When a reservation does
// not fit, the wave raises `flag` and waits at a rendezvous; every other wave joins at its next
// checkpoint (it polls `flag` once per group) or when it has run out of work, and the whole
// workgroup prunes the pool together: two 1024-bin histogram passes over the top 20 bits of the
// ordered scores find the smallest bucket with k candidates at or below it, everything above is
// dropped and the bound tightens to the top of that bucket.
//
// Protocol (each wave executes the same number of barriers):
//   scanning wave:  if (poll()) rendezvous();  ...  while (!try_push(...)) rendezvous();
//   finished wave:  finish_wave();  while (!rendezvous()) {}
// rendezvous() returns true once every wave has called finish_wave().
struct BlockPoolCtl {
    int count;      // reserved entries (may run past cap once a reservation failed)
    int valid_end;  // entries [0, min(count, valid_end)) are written
    int flag;       // a reservation failed: prune at the next rendezvous
    int done;       // waves that have finished their work
    int kept;
    int bin;        // histogram search result
    int below;      // candidates in bins before `bin`
    float bound;
    key_t bound_key;   // kEmptyKey, or the k-th smallest key once ties at the k-th score overflowed the pool
};

template <int W>
struct BlockPool {
    static constexpr int NT = W * kWave;
    static constexpr int kMaxPerThread = W >= 16 ? 4 : 8;   // cap <= kMaxPerThread * NT
    // Every pointer SAYS that it is an LDS address.  Through generic pointers the compiler emits flat
    // instructions, which count as vector-memory operations as well: with one anywhere in the scan loop (the
    // poll of `flag`, a prune) it can no longer tell a pending flat access from the codes of the next group that
    // were requested a moment ago, waits for everything before it evaluates the current group, and the scan runs
    // at one memory latency per group.
    typedef __attribute__((address_space(3))) key_t lds_key_t;
    typedef __attribute__((address_space(3))) int lds_int_t;
    typedef __attribute__((address_space(3))) BlockPoolCtl lds_ctl_t;
    lds_key_t *buf;
    lds_int_t *hist;           // 1024 ints
    volatile lds_ctl_t *ctl;
    int cap, k;
    static __device__ __forceinline__ int lds_add(volatile lds_int_t *p, int v)
    {
        return __hip_atomic_fetch_add((lds_int_t *)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    float bound;               // wave-uniform copy of ctl->bound
    key_t bound_key;           // wave-uniform copy of ctl->bound_key

    // All threads call; a __syncthreads() must follow before the first push.
    __device__ __forceinline__ void init(key_t *b, int cap_, int k_, int *hist_, BlockPoolCtl *c, int tid)
    {
        buf = (lds_key_t *)b;
        cap = cap_;
        k = k_;
        hist = (lds_int_t *)hist_;
        ctl = (volatile lds_ctl_t *)c;
        bound = __builtin_inff();
        bound_key = kEmptyKey;
        if (tid == 0) {
            c->bound_key = kEmptyKey;
            c->count = 0;
            c->valid_end = cap_;
            c->flag = 0;
            c->done = 0;
            c->kept = 0;
            c->bound = __builtin_inff();
        }
    }

    __device__ __forceinline__ bool poll() const { return __builtin_amdgcn_readfirstlane(ctl->flag) != 0; }   // ds_read

    // All lanes of the wave call.  False: the pool is full -- call rendezvous(), re-test the
    // candidates against the new bound and try again.
    __device__ __forceinline__ bool try_push(bool pass, float score, uint32_t idx, int lane)
    {
        unsigned long long mask = __ballot(pass);
        if (mask == 0) {
            return true;
        }
        if (bound_key != kEmptyKey) {
            pass = pass && make_key(score, idx) < bound_key;
            mask = __ballot(pass);
            if (mask == 0) {
                return true;
            }
        }
        const int n = __popcll(mask);
        const int pre = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        int base = 0;
        if (lane == 0) {
            base = lds_add(&ctl->count, n);
        }
        base = __builtin_amdgcn_readfirstlane(base);
        if (base + n <= cap) {
            if (pass) {
                buf[base + pre] = make_key(score, idx);
            }
            return true;
        }
        if (lane == 0) {
            if (base < cap) {
                ctl->valid_end = base;   // the one reservation that straddles the end
            }
            ctl->flag = 1;
        }
        return false;
    }

    __device__ __forceinline__ void finish_wave(int lane)
    {
        if (lane == 0) {
            lds_add(&ctl->done, 1);
        }
    }

    __device__ __forceinline__ int size() const
    {
        const int c = ctl->count, v = ctl->valid_end;
        return c < v ? c : v;
    }

    // Wave 0: first bin whose inclusive prefix count reaches `rank` (1 <= rank <= total).
    __device__ inline void find_bin(int rank, int tid)
    {
        if (tid < kWave) {
            int part = 0;
            for (int j = 0; j < 16; j++) {
                part += hist[tid * 16 + j];
            }
            int incl = part;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const int up = __shfl_up(incl, o);
                if (tid >= o) {
                    incl += up;
                }
            }
            const unsigned long long reach = __ballot(incl >= rank);
            const int owner = reach ? __builtin_ctzll(reach) : kWave - 1;
            if (tid == owner) {
                int run = incl - part, bin = tid * 16 + 15;
                for (int j = 0; j < 16; j++) {
                    if (run + hist[tid * 16 + j] >= rank) {
                        bin = tid * 16 + j;
                        break;
                    }
                    run += hist[tid * 16 + j];
                }
                ctl->bin = bin;
                ctl->below = run;
            }
        }
    }

    // All NT threads: drop what cannot be among the k best, tighten the bound, reopen the pool.
    __device__ inline void prune(int tid)
    {
        constexpr int SH = 32 - kSelectBits;
        const int lane = tid & 63;
        const int n = size();
        key_t e[kMaxPerThread];
#pragma unroll
        for (int j = 0; j < kMaxPerThread; j++) {
            const int i = j * NT + tid;
            e[j] = i < n ? buf[i] : kEmptyKey;
        }
        uint32_t P = 0xffffffffu >> SH;   // keep everything unless k candidates exist
        if (n >= k) {
            for (int i = tid; i < 1024; i += NT) {
                hist[i] = 0;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < kMaxPerThread; j++) {
                if (e[j] != kEmptyKey) {
                    lds_add(&hist[(uint32_t)(e[j] >> (32 + SH + 10))], 1);
                }
            }
            __syncthreads();
            find_bin(k, tid);
            __syncthreads();
            const uint32_t b1 = (uint32_t)ctl->bin;
            const int rank2 = k - ctl->below;
            __syncthreads();
            for (int i = tid; i < 1024; i += NT) {
                hist[i] = 0;
            }
            __syncthreads();
#pragma unroll
            for (int j = 0; j < kMaxPerThread; j++) {
                const uint32_t pre = (uint32_t)(e[j] >> (32 + SH));
                if (e[j] != kEmptyKey && (pre >> 10) == b1) {
                    lds_add(&hist[pre & 1023u], 1);
                }
            }
            __syncthreads();
            find_bin(rank2, tid);
            __syncthreads();
            P = (b1 << 10) | (uint32_t)ctl->bin;
        }
        if (tid == 0) {
            ctl->kept = 0;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < kMaxPerThread; j++) {
            const bool keep = e[j] != kEmptyKey && (uint32_t)(e[j] >> (32 + SH)) <= P;
            const unsigned long long mask = __ballot(keep);
            if (mask) {
                const int pre =
                    __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                int base = 0;
                if (lane == 0) {
                    base = lds_add(&ctl->kept, __popcll(mask));
                }
                base = __builtin_amdgcn_readfirstlane(base);
                if (keep) {
                    buf[base + pre] = e[j];
                }
            }
        }
        __syncthreads();
        int kept = ctl->kept;
        float top = ScoreOps<float>::bucket_top((P << SH) | ((1u << SH) - 1u));
        if (kept > cap - NT) {
            // one bucket holds almost everything: exact selection by sorting
            for (int i = kept + tid; i < cap; i += NT) {
                buf[i] = kEmptyKey;
            }
            block_bitonic_sort((key_t *)buf, cap, tid, NT);
            kept = k;
            top = key_score(buf[k - 1]);
            if (tid == 0) {
                ctl->bound_key = buf[k - 1];
            }
        }
        __syncthreads();
        if (tid == 0) {
            const float b = ctl->bound;
            ctl->bound = (n >= k && top < b) ? top : b;
            ctl->count = kept;
            ctl->valid_end = cap;
            ctl->flag = 0;
        }
        __syncthreads();
    }

    // All waves of the workgroup meet here.  True once every wave has finished its work.
    __device__ inline bool rendezvous(int tid)
    {
        __syncthreads();
        const int f = ctl->flag, d = ctl->done;
        __syncthreads();
        if (f) {
            prune(tid);
        }
        bound = wave_uniform(ctl->bound);
        bound_key = wave_uniform_key(ctl->bound_key);
        return d == W;
    }

    // After the last rendezvous: sorts the pool ascending in place, returns the number of keys.  Only the
    // smallest power of two that holds them is sorted (a pool pruned to little more than k is far from full).
    __device__ inline int sort_all(int tid)
    {
        const int n = size();
        int n2 = 2;
        while (n2 < n) {
            n2 <<= 1;
        }
        __syncthreads();
        for (int i = n + tid; i < n2; i += NT) {
            buf[i] = kEmptyKey;
        }
        block_bitonic_sort((key_t *)buf, n2, tid, NT);
        return n;
    }
};

inline int block_pool_capacity(int k, int waves)
{
    int cap = 1024;
    while (cap < k + 2 * waves * kWave) {
        cap <<= 1;
    }
    return cap;
}

inline int wave_pool_capacity(int k)
{
    int cap = 256;
    while (cap < k + 2 * kWave) {
        cap <<= 1;
    }
    return cap;
}

}  // namespace ixa
