// Persistent "ring" score kernels: query x base score tiles at matrix-core rate.
//
// A K-step of MFMAs lasts a few hundred (int8) to a few thousand (fp32) cycles, and a tile of the
// headline shapes has only 8 K-steps, so a kernel that starts and drains a pipeline per tile spends
// a large share of its time waiting for the first operands.  Here instead
//   * a workgroup is persistent and walks a list of 256 x 128 tiles; the stream of K-steps (64 bytes
//     of every operand row each) runs continuously across tile boundaries;
//   * operands go from global memory straight into LDS (global_load_lds_dwordx4, no VGPR staging)
//     into a ring of kStages buffers, kStages - 1 steps ahead of the MFMAs; completion is tracked
//     with s_waitcnt vmcnt + s_barrier, without the full memory fence of __syncthreads();
//   * each wavefront owns 128 x 64 of the tile (4 x 2 blocks of 32 x 32), so one operand fragment
//     read from LDS feeds 1.33 MFMA blocks on average;
//   * rows are stored unpadded (64 bytes per row and step); the 16-byte chunk index is XOR-swizzled
//     with bits 2-3 of the row, which makes the 128-bit fragment reads of 16 consecutive rows hit
//     16 different bank groups;
//   * tiles are dealt so that all workgroups of an XCD work on the same base tile at the same time
//     (it is fetched from HBM once and re-used out of that XCD's L2);
//   * two workgroups share a CU, so one's epilogue overlaps the other's MFMAs.
// Scores: int8 -> exact int32 |q|^2 + |b|^2 - 2 q.b (v_mfma_i32_32x32x32_i8);
//         fp32 -> (|q|^2 + |b|^2) - g - g or -g (v_mfma_f32_32x32x2_f32).
// The sum over k is order-free for integers, and for fp32 any fixed k-assignment that is the same
// for both operands is a valid accumulation order, so each lane half owns half of a K-step.
#include "coarse.h"
#include "topk.h"

namespace ixa {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kRingTM = 256, kRingTN = 128, kRingRows = kRingTM + kRingTN;
constexpr int kRingStageBytes = kRingRows * 64;
constexpr int kRingStages = 3;
constexpr int kRingAuxBytes = 1280;   // per-wave staging of a filtered epilogue's operands
constexpr int kRingLoadsPerWave = kRingRows / 16 / 4;  // wave-wide 1 KB loads per stage and wavefront

struct I8Traits {
    using T = int8_t;
    using S = int32_t;
    using Acc = v16i;
    static constexpr int kElemsPerStep = 64;
    // one K-step = 2 sub-steps of 32 bytes; a lane half owns 16 of them
    template <bool SWAP, bool ZERO>
    static __device__ __forceinline__ void mma(const unsigned char *stage, int wr, int wc, int l32, int half,
                                               Acc (&acc)[4][2])
    {
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int c = kk * 2 + half;
            v4i a[4], b[2];
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                const int r = wr * 128 + ra * 32 + l32;
                a[ra] = *reinterpret_cast<const v4i *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const int r = kRingTM + wc * 64 + rb * 32 + l32;
                b[rb] = *reinterpret_cast<const v4i *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const Acc c0 = (ZERO && kk == 0) ? Acc{} : acc[ra][rb];   // a tile's first product starts from zero
                    acc[ra][rb] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b[rb], a[ra], c0, 0, 0, 0)
                                       : __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ra], b[rb], c0, 0, 0, 0);
                }
            }
        }
    }
};

// bf16 operands, fp32 accumulation (v_mfma_f32_32x32x16_bf16): same data movement as int8.
struct Bf16Traits {
    using T = uint16_t;
    using S = float;
    using Acc = v16f;
    static constexpr int kElemsPerStep = 32;
    template <bool SWAP, bool ZERO>
    static __device__ __forceinline__ void mma(const unsigned char *stage, int wr, int wc, int l32, int half,
                                               Acc (&acc)[4][2])
    {
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int c = kk * 2 + half;
            bf16x8 a[4], b[2];
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                const int r = wr * 128 + ra * 32 + l32;
                a[ra] = *reinterpret_cast<const bf16x8 *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const int r = kRingTM + wc * 64 + rb * 32 + l32;
                b[rb] = *reinterpret_cast<const bf16x8 *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const Acc c0 = (ZERO && kk == 0) ? Acc{} : acc[ra][rb];
                    acc[ra][rb] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[rb], a[ra], c0, 0, 0, 0)
                                       : __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ra], b[rb], c0, 0, 0, 0);
                }
            }
        }
    }
};

struct F32Traits {
    using T = float;
    using S = float;
    using Acc = v16f;
    static constexpr int kElemsPerStep = 16;
    // one K-step = 16 floats; a lane half owns 8 of them (two 16-byte chunks) and feeds them to 8
    // consecutive 32x32x2 MFMAs
    template <bool SWAP, bool ZERO>
    static __device__ __forceinline__ void mma(const unsigned char *stage, int wr, int wc, int l32, int half,
                                               Acc (&acc)[4][2])
    {
        v4f a[4][2], b[2][2];
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
            const int c = half * 2 + cc;
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                const int r = wr * 128 + ra * 32 + l32;
                a[ra][cc] = *reinterpret_cast<const v4f *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const int r = kRingTM + wc * 64 + rb * 32 + l32;
                b[rb][cc] = *reinterpret_cast<const v4f *>(stage + r * 64 + ((c ^ ((r >> 2) & 3)) << 4));
            }
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const float av = a[ra][t >> 2][t & 3], bv = b[rb][t >> 2][t & 3];
                    const Acc c0 = (ZERO && t == 0) ? Acc{} : acc[ra][rb];
                    acc[ra][rb] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x2f32(bv, av, c0, 0, 0, 0)
                                       : __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, c0, 0, 0, 0);
                }
            }
        }
    }
};

template <typename Tr, bool FILTER>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void score_ring_kernel(
    const typename Tr::T *__restrict__ Q, int64_t nq, const typename Tr::T *__restrict__ B, int64_t nb, int d,
    const typename Tr::S *__restrict__ qn, const typename Tr::S *__restrict__ bn, int metric,
    typename Tr::S *__restrict__ out, int64_t ldo, int tiles_m, int tiles_n, ScoreFilter<typename Tr::S> flt)
{
    using T = typename Tr::T;
    using S = typename Tr::S;
    constexpr bool kInt = sizeof(T) == 1;
    extern __shared__ __align__(16) unsigned char ring[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1, wc = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    const int nk = d / Tr::kElemsPerStep;
    const int64_t row_bytes = (int64_t)d * sizeof(T);

    // work list: XCD x owns base tiles x, x + 8, ...; its workgroups take (base tile, query tile)
    // pairs round-robin, query tile fastest
    const int xcd = blockIdx.x & 7, wi = blockIdx.x >> 3, wpx = gridDim.x >> 3;
    const int own_n = tiles_n > xcd ? (tiles_n - xcd + 7) / 8 : 0;
    const int64_t items = (int64_t)own_n * tiles_m;
    const int my_items = items > wi ? (int)((items - wi + wpx - 1) / wpx) : 0;
    const int total = my_items * nk;
    if (total == 0) {
        return;
    }
    auto item_tile = [&](int it, int64_t &tm, int64_t &tn) {
        const uint32_t t = (uint32_t)wi + (uint32_t)it * (uint32_t)wpx;
        tn = xcd + 8 * (int64_t)(t / (uint32_t)tiles_m);
        tm = t % (uint32_t)tiles_m;
    };
    const unsigned char *Qb = reinterpret_cast<const unsigned char *>(Q);
    const unsigned char *Bb = reinterpret_cast<const unsigned char *>(B);

    // Per-lane source pointers of the tile whose K-steps are being issued (recomputed once per
    // tile); a K-step then only adds ks * 64 bytes.
    const unsigned char *src[kRingLoadsPerWave];
    auto set_sources = [&](int it) {
        int64_t tm, tn;
        item_tile(it, tm, tn);
#pragma unroll
        for (int j = 0; j < kRingLoadsPerWave; j++) {
            const int rg = wave * kRingLoadsPerWave + j;          // group of 16 stage rows
            const int row = rg * 16 + (lane >> 2);                // stage row: 0..255 queries, 256..383 base
            const int chunk = (lane & 3) ^ ((row >> 2) & 3);
            if (rg < kRingTM / 16) {
                int64_t r = tm * kRingTM + row;
                r = r < nq ? r : nq - 1;
                src[j] = Qb + r * row_bytes + chunk * 16;
            } else {
                int64_t r = tn * kRingTN + (row - kRingTM);
                r = r < nb ? r : nb - 1;
                src[j] = Bb + r * row_bytes + chunk * 16;
            }
        }
    };
    // issue the loads of one K-step (step ks of the current issue tile) into ring buffer `slot`
    auto issue = [&](int ks, int slot) {
        unsigned char *stage = ring + slot * kRingStageBytes;
#pragma unroll
        for (int j = 0; j < kRingLoadsPerWave; j++) {
            const int rg = wave * kRingLoadsPerWave + j;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src[j] + ks * 64),
                                             (__attribute__((address_space(3))) void *)(stage + rg * 1024), 16, 0, 0);
        }
    };

    typename Tr::Acc acc[4][2];   // written from zero by the first K-step of every tile

    // (item, step, ring slot) of the next K-step to issue and of the one being computed
    int issued = 0, i_it = 0, i_ks = 0, i_slot = 0;
    auto issue_next = [&]() {
        if (i_ks == 0) {
            set_sources(i_it);
        }
        issue(i_ks, i_slot);
        issued++;
        i_slot = i_slot + 1 == kRingStages ? 0 : i_slot + 1;
        if (++i_ks == nk) {
            i_ks = 0;
            i_it++;
        }
    };
    while (issued < kRingStages - 1 && issued < total) {
        issue_next();
    }
    int c_it = 0, c_ks = 0, c_slot = 0;
    bool stored = false;  // the previous iteration ended with an epilogue that issued stores

    // Filtered launches stage what the epilogue of a tile needs -- the base norms of the wave's 64
    // columns and the bounds (and norms) of its 128 query rows -- in a small per-wave LDS area, with
    // the same global->LDS loads as the ring and one K-step ahead, so the epilogue never waits for
    // memory and the main loop carries no registers for it.  The s_waitcnt immediates below count
    // these loads (kPrefetchLoads per wave).
    //   aux +   0: 64 base norms      (lanes 0..15, 16 bytes each)
    //   aux + 256: 128 tau or thr     (lanes 16..47)
    //   aux + 768: 128 query norms    (lanes 0..31 of a second load; fp32 scores only)
    constexpr int kPrefetchLoads = kInt ? 1 : 2;
    unsigned char *aux = ring + kRingStages * kRingStageBytes + wave * kRingAuxBytes;
    const S *bound = kInt ? flt.thr : flt.tau;
    const bool prefetch = FILTER && nk >= 2 && nb % 4 == 0 && nq % 4 == 0 && bn != nullptr && qn != nullptr &&
                          bound != nullptr && reinterpret_cast<uintptr_t>(bn) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(qn) % 16 == 0 && reinterpret_cast<uintptr_t>(bound) % 16 == 0;
    bool fetched = false;   // the previous iteration issued the fetch
    auto fetch_epilogue_operands = [&](int it) {
        int64_t tm, tn;
        item_tile(it, tm, tn);
        const int64_t i0 = tm * kRingTM, j0 = tn * kRingTN;
        asm volatile("" ::: "memory");
        if (lane < 48) {
            // groups of four that start past the end read group 0 instead; their scores are rejected
            // by index in the epilogue
            const S *p;
            if (lane < 16) {
                const int64_t col = j0 + wc * 64 + lane * 4;
                p = bn + (col < nb ? col : 0);
            } else {
                const int64_t row = i0 + wr * 128 + (lane - 16) * 4;
                p = bound + (row < nq ? row : 0);
            }
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                             (__attribute__((address_space(3))) void *)aux, 16, 0, 0);
        }
        if constexpr (!kInt) {
            if (lane < 32) {
                const int64_t row = i0 + wr * 128 + lane * 4;
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(qn + (row < nq ? row : 0)),
                                                 (__attribute__((address_space(3))) void *)(aux + 768), 16, 0, 0);
            }
        }
        asm volatile("" ::: "memory");
    };
    for (int g = 0; g < total; g++) {
        // The loads of step g must have landed; later steps may still be in flight.  vmcnt counts
        // loads and stores in issue order, so right after a storing epilogue the usual count would
        // also wait for all of its (much younger) stores; 63 is the largest expressible count and
        // still covers the loads of step g, which are older than every store.
        if (!FILTER && stored && issued - g - 1 >= kRingStages - 2) {
            __builtin_amdgcn_s_waitcnt(0xcf7f);   // vmcnt(63): covers the <= 32 + 6 younger operations
        } else if (issued - g - 1 >= kRingStages - 2) {
            constexpr int kInFlight = (kRingStages - 2) * kRingLoadsPerWave;
            if (FILTER && fetched) {
                // queue: [step g][step g + 1][epilogue fetch]; only step g has to be complete
                constexpr int n = kInFlight + kPrefetchLoads;
                __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
            } else {
                __builtin_amdgcn_s_waitcnt(0x0f70 | kInFlight);
            }
        } else {
            __builtin_amdgcn_s_waitcnt(0x0f70);
        }
        stored = false;
        fetched = false;
        __builtin_amdgcn_s_barrier();
        const bool issued_now = issued < total;
        if (issued_now) {
            issue_next();  // goes into the buffer that step g - 1 has just finished reading
        }
        if (FILTER && prefetch && c_ks == nk - 2) {
            fetch_epilogue_operands(c_it);
            fetched = true;
        }
        if (c_ks == 0) {
            Tr::template mma<FILTER, true>(ring + c_slot * kRingStageBytes, wr, wc, l32, half, acc);
        } else {
            Tr::template mma<FILTER, false>(ring + c_slot * kRingStageBytes, wr, wc, l32, half, acc);
        }
        const bool last_step = c_ks == nk - 1;
        const int done_it = c_it;
        c_slot = c_slot + 1 == kRingStages ? 0 : c_slot + 1;
        if (++c_ks == nk) {
            c_ks = 0;
            c_it++;
        }
        // Two epilogues.  Filtered launches make the BASE fragment the first MFMA operand, so a lane
        // owns one query row per block (its bound is a per-lane scalar) -- cheapest test per score.
        // Storing launches keep the query fragment first: a lane owns one base column and 32 lanes
        // write 128 contiguous bytes of a score row, which is what the memory system wants.
        if (FILTER && last_step) {
            // The base fragment is the first MFMA operand, so in accumulator block (ra, rb) a lane
            // owns ONE query row (ra * 32 + l32) and its 16 registers are base columns
            // rb * 32 + 8 * (r / 4) + 4 * half + (r % 4): four runs of four consecutive columns.
            // Per-query values are per-lane scalars and results leave as 128-bit stores.
            int64_t tm, tn;
            item_tile(done_it, tm, tn);
            const int64_t i0 = tm * kRingTM, j0 = tn * kRingTN;
            const bool vec_out = !FILTER && (ldo % 4 == 0) && (reinterpret_cast<uintptr_t>(out) % 16 == 0);
            // the base norms of this lane's 32 columns: out of the staging area, or loaded here
            S bnq[2][4][4];
            const bool use_bn = kInt || metric == kMetricL2;
            const bool vec_bn = reinterpret_cast<uintptr_t>(bn) % 16 == 0;
            if (prefetch) {
                // the staging loads are older than the K-step loads issued in this iteration
                if (issued_now) {
                    __builtin_amdgcn_s_waitcnt(0x0f70 | kRingLoadsPerWave);
                } else {
                    __builtin_amdgcn_s_waitcnt(0x0f70);
                }
                asm volatile("" ::: "memory");
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
#pragma unroll
                    for (int rq = 0; rq < 4; rq++) {
                        const uint4 u = *reinterpret_cast<const uint4 *>(aux + (rb * 32 + 8 * rq + 4 * half) * 4);
                        bnq[rb][rq][0] = __builtin_bit_cast(S, u.x);
                        bnq[rb][rq][1] = __builtin_bit_cast(S, u.y);
                        bnq[rb][rq][2] = __builtin_bit_cast(S, u.z);
                        bnq[rb][rq][3] = __builtin_bit_cast(S, u.w);
                    }
                }
            }
#pragma unroll
            for (int rb = 0; rb < 2 && !prefetch; rb++) {
#pragma unroll
                for (int rq = 0; rq < 4; rq++) {
                    const int64_t col = j0 + wc * 64 + rb * 32 + 8 * rq + 4 * half;
                    if (use_bn && vec_bn && col + 3 < nb) {
                        const uint4 u = *reinterpret_cast<const uint4 *>(bn + col);
                        bnq[rb][rq][0] = __builtin_bit_cast(S, u.x);
                        bnq[rb][rq][1] = __builtin_bit_cast(S, u.y);
                        bnq[rb][rq][2] = __builtin_bit_cast(S, u.z);
                        bnq[rb][rq][3] = __builtin_bit_cast(S, u.w);
                    } else {
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            bnq[rb][rq][t] = (use_bn && col + t < nb) ? bn[col + t] : (S)0;
                        }
                    }
                }
            }
            if constexpr (kInt) {
                // -|b|^2, so that a score's test value is one shift-add: 2 q.b - |b|^2
#pragma unroll
                for (int t = 0; t < 32; t++) {
                    bnq[t >> 4][(t >> 2) & 3][t & 3] = -bnq[t >> 4][(t >> 2) & 3][t & 3];
                }
            }
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                asm volatile("" ::: "memory");   // one query block at a time keeps register pressure low
                const int64_t row = i0 + wr * 128 + ra * 32 + l32;
                const bool row_ok = row < nq;
                S rowv, tauv;
                if (prefetch) {
                    const S bv = *reinterpret_cast<const S *>(aux + 256 + (ra * 32 + l32) * 4);
                    rowv = kInt ? bv : *reinterpret_cast<const S *>(aux + 768 + (ra * 32 + l32) * 4);
                    tauv = kInt ? (S)0 : bv;
                } else if (kInt) {
                    // |b|^2 - 2 q.b <= tau - |q|^2  <=>  distance <= tau (exact in integers)
                    rowv = row_ok ? flt.thr[row] : (S)0x80000000;
                    tauv = 0;
                } else {
                    rowv = (row_ok && metric == kMetricL2) ? qn[row] : (S)0;
                    tauv = row_ok ? flt.tau[row] : (S)(-__builtin_inff());
                }
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    // all 16 scores of the block first, then ONE test of their minimum against the
                    // lane's bound: admissions are rare, so the per-score path almost never runs
                    S v[16];
                    S best = ScoreOps<S>::worst();
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const S bnv = bnq[rb][r >> 2][r & 3];
                        if constexpr (kInt) {
                            // bnq holds -|b|^2: v = -(distance - |q|^2) in one shift-add, largest is best
                            v[r] = (S)(((uint32_t)acc[ra][rb][r] << 1) + (uint32_t)bnv);
                            best = (r == 0 || v[r] > best) ? v[r] : best;
                            continue;
                        } else {
                            const float g = acc[ra][rb][r];
                            if (metric == kMetricL2) {
                                float w = __fadd_rn(rowv, bnv);
                                w = __fsub_rn(w, g);
                                v[r] = __fsub_rn(w, g);
                            } else {
                                v[r] = -g;
                            }
                        }
                        best = v[r] < best ? v[r] : best;
                    }
                    const S lane_bound = kInt ? rowv : tauv;
                    if constexpr (kInt) {
                        best = -best;
                    }
                    if (__ballot(row_ok && best <= lane_bound)) {
                        // opaque to the optimiser here, or it keeps all 32 column offsets of this rare
                        // path in registers across the whole main loop
                        int cb = wc * 64 + rb * 32 + 4 * half;
                        asm volatile("" : "+v"(cb));
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int64_t col = j0 + cb + 8 * (r >> 2) + (r & 3);
                            const S part = kInt ? -v[r] : v[r];
                            if (row_ok && part <= lane_bound && col < nb) {
                                S val = part;
                                if constexpr (kInt) {
                                    val += qn[row];
                                }
                                const int pos = atomicAdd(&flt.cnt[row], 1);
                                if (pos < flt.cap) {
                                    flt.cand[row * flt.cap + pos] = make_key(val, (uint32_t)(col + flt.col_base));
                                }
                            }
                        }
                    }
                }
            }
        }
        if (!FILTER && last_step) {
            stored = true;
            int64_t tm, tn;
            item_tile(done_it, tm, tn);
            const int64_t i0 = tm * kRingTM, j0 = tn * kRingTN;
            S bnv[2];
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const int64_t col = j0 + wc * 64 + rb * 32 + l32;
                bnv[rb] = (col < nb && (kInt || metric == kMetricL2)) ? bn[col] : (S)0;
            }
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                // one 32-row block at a time keeps the per-row operands of only 16 rows live
                asm volatile("" ::: "memory");
                S rowv[16];   // int8 + FILTER: tau - |q|^2; otherwise |q|^2
                S tauv[16];   // fp32 + FILTER: tau
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int64_t row = i0 + wr * 128 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    if (kInt) {
                        // |b|^2 - 2 q.b <= tau - |q|^2  <=>  distance <= tau (exact in integers)
                        rowv[r] = row < nq ? (FILTER ? flt.thr[row] : qn[row]) : (FILTER ? (S)0x80000000 : (S)0);
                    } else {
                        rowv[r] = (row < nq && metric == kMetricL2) ? qn[row] : (S)0;
                        tauv[r] = (FILTER && row < nq) ? flt.tau[row] : (S)(-__builtin_inff());
                    }
                }
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const int64_t col = j0 + wc * 64 + rb * 32 + l32;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int64_t row = i0 + wr * 128 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                        S v;
                        bool admit;
                        if constexpr (kInt) {
                            const S part = bnv[rb] - 2 * acc[ra][rb][r];
                            admit = part <= rowv[r];
                            v = FILTER ? part : part + rowv[r];
                        } else {
                            const float g = acc[ra][rb][r];
                            if (metric == kMetricL2) {
                                v = __fadd_rn(rowv[r], bnv[rb]);
                                v = __fsub_rn(v, g);
                                v = __fsub_rn(v, g);
                            } else {
                                v = -g;
                            }
                            admit = v <= tauv[r];
                        }
                        if (FILTER) {
                            if (admit && col < nb) {
                                if constexpr (kInt) {
                                    v += qn[row];
                                }
                                const int pos = atomicAdd(&flt.cnt[row], 1);
                                if (pos < flt.cap) {
                                    flt.cand[row * flt.cap + pos] = make_key(v, (uint32_t)(col + flt.col_base));
                                }
                            }
                        } else if (row < nq && col < nb) {
                            out[row * ldo + col] = v;
                        }
                    }
                }
            }
        }
    }
}

template <typename Tr>
bool launch_ring(const typename Tr::T *Q, int64_t nq, const typename Tr::T *B, int64_t nb, int d,
                 const typename Tr::S *qn, const typename Tr::S *bn, int metric, typename Tr::S *out, int64_t ldo,
                 bool filter, ScoreFilter<typename Tr::S> flt, hipStream_t s)
{
    if (d % Tr::kElemsPerStep != 0 || nb < 8 * kRingTN || reinterpret_cast<uintptr_t>(Q) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(B) % 16 != 0) {
        return false;
    }
    const int64_t rt_m = (nq + kRingTM - 1) / kRingTM, rt_n = (nb + kRingTN - 1) / kRingTN;
    if (rt_m * rt_n >= ((int64_t)1 << 31) || rt_m * ((rt_n + 7) / 8) * (d / Tr::kElemsPerStep) >= ((int64_t)1 << 30)) {
        return false;
    }
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        IXA_HIP(hipGetDevice(&dev));
        IXA_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    }
    const unsigned grid = (unsigned)((2 * cus + 7) / 8 * 8);   // two persistent workgroups per CU
    const size_t smem = (size_t)kRingStages * kRingStageBytes + (filter ? 4 * kRingAuxBytes : 0);
    if (filter) {
        auto kern = score_ring_kernel<Tr, true>;
        IXA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, s, Q, nq, B, nb, d, qn, bn, metric, out, ldo, (int)rt_m,
                           (int)rt_n, flt);
    } else {
        auto kern = score_ring_kernel<Tr, false>;
        IXA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, s, Q, nq, B, nb, d, qn, bn, metric, out, ldo, (int)rt_m,
                           (int)rt_n, flt);
    }
    return true;
}

}  // namespace

bool launch_score_ring_i8(const int8_t *Q, int64_t nq, const int8_t *B, int64_t nb, int d, const int32_t *qn,
                          const int32_t *bn, int32_t *out, int64_t ldo, bool filter, ScoreFilter<int32_t> flt,
                          hipStream_t s)
{
    return launch_ring<I8Traits>(Q, nq, B, nb, d, qn, bn, kMetricL2, out, ldo, filter, flt, s);
}

bool launch_score_ring_bf16(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                            const float *bn, int metric, float *out, int64_t ldo, bool filter, ScoreFilter<float> flt,
                            hipStream_t s)
{
    return launch_ring<Bf16Traits>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, filter, flt, s);
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

__global__ __launch_bounds__(256) void split_bf16x3_kernel(const float *__restrict__ x, int64_t n, int d, int dp,
                                                           int base_side, uint16_t *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
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

void launch_split_bf16x3(const float *x, int64_t n, int d, int dp, bool base_side, uint16_t *out, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(split_bf16x3_kernel, dim3((unsigned)((n * dp + 255) / 256)), dim3(256), 0, s, x, n, d, dp,
                           base_side ? 1 : 0, out);
    }
}

// Raises *flag unless, for every query, no centroid outside its approximate candidate list can beat
// its nout-th exact score: (approximate score of the last candidate) - err > (nout-th exact score),
// err = err_scale * |q| * max|c| + round_scale * (|q| + max|c|)^2.  Rows whose candidate list is not full hold every centroid.
__global__ __launch_bounds__(256) void verify_superset_kernel(const key_t *__restrict__ running, int ncand,
                                                              const float *__restrict__ exact_dist, int nout,
                                                              const float *__restrict__ qn, float cmax, float err_scale,
                                                              float round_scale, int metric, int64_t nq,
                                                              int *__restrict__ flag)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= nq) {
        return;
    }
    const key_t last = running[i * ncand + (ncand - 1)];
    if (last == kEmptyKey) {
        return;
    }
    const float a_last = key_score(last);
    const float d_out = exact_dist[i * nout + (nout - 1)];
    const float s_star = metric == kMetricL2 ? d_out : -d_out;
    const float qlen = sqrtf(qn[i]);
    const float err = err_scale * qlen * cmax + round_scale * (qlen + cmax) * (qlen + cmax);
    if (!(a_last - err > s_star)) {
        *flag = 1;
    }
}

void launch_verify_superset(const unsigned long long *running, int ncand, const float *exact_dist, int nout,
                            const float *qn, float cmax, float err_scale, float round_scale, int metric, int64_t nq,
                            int *flag, hipStream_t s)
{
    if (nq > 0) {
        hipLaunchKernelGGL(verify_superset_kernel, dim3((unsigned)((nq + 255) / 256)), dim3(256), 0, s, running, ncand,
                           exact_dist, nout, qn, cmax, err_scale, round_scale, metric, nq, flag);
    }
}

bool launch_score_ring_f32(const float *Q, int64_t nq, const float *B, int64_t nb, int d, const float *qn,
                           const float *bn, int metric, float *out, int64_t ldo, bool filter, ScoreFilter<float> flt,
                           hipStream_t s)
{
    return launch_ring<F32Traits>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, filter, flt, s);
}

}  // namespace ixa
