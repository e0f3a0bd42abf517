// Persistent "ring" score kernels: query x base score tiles at matrix-core rate.
//
// A K-step of MFMAs lasts a few hundred (bf16) to a few thousand (fp32) cycles, and a tile of the
// headline shapes has only 8 K-steps, so a kernel that starts and drains a pipeline per tile spends
// a large share of its time waiting for the first operands.  Here instead
//   * a workgroup of 8 wavefronts is persistent (one per CU) and walks a list of 256 x 256 tiles; the
//     stream of K-steps (64 bytes of every operand row each) runs continuously across tile
//     boundaries.  The square tile stages 512 rows for 65536 products per K-element: the L2 -> LDS
//     traffic, which bounds the bf16 variant, is 2/3 of what a 256 x 128 tile needs;
//   * operands go from global memory straight into LDS (global_load_lds_dwordx4, no VGPR staging)
//     into a ring of kRingStages buffers, two to three steps ahead of the MFMAs; completion is
//     tracked with s_waitcnt vmcnt + s_barrier, without the full memory fence of __syncthreads();
//   * each wavefront owns 128 x 64 of the tile (4 x 2 blocks of 32 x 32), so one operand fragment
//     read from LDS feeds 1.33 MFMA blocks on average;
//   * a K-step is consumed as two half-steps with two fragment register sets: the LDS reads of the
//     next half-step are issued before the MFMAs of the current one, and the once-per-step barrier
//     sits between the two half-steps of a stage, so no wave ever waits for LDS in front of idle
//     matrix cores;
//   * rows are stored unpadded (64 bytes per row and step); the 16-byte chunk index is XOR-swizzled
//     with bits 2-3 of the row, which makes the 128-bit fragment reads of 16 consecutive rows hit
//     16 different bank groups;
//   * tiles are dealt so that all workgroups of an XCD work on the same base tile at the same time
//     (it is fetched from HBM once and re-used out of that XCD's L2).
// Scores: bf16 -> fp32 accumulation (v_mfma_f32_32x32x16_bf16);
//         fp32 -> (|q|^2 + |b|^2) - g - g or -g (v_mfma_f32_32x32x2_f32).
// Any fixed k-assignment that is the same for both operands is a valid accumulation order, so each lane
// half owns half of a K-step.  (int8 Flat has a kernel of its own: flat_i8.hip.)
#include <type_traits>

#include "coarse.h"
#include "topk.h"

namespace ixa {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kRingWaves = 8;
constexpr int kRingTM = 256, kRingTN = 256, kRingRows = kRingTM + kRingTN;
constexpr int kRingStageBytes = kRingRows * 64;
constexpr int kRingStages = 3;
constexpr int kRingAuxBytes = 1280;   // per-wave staging of a filtered epilogue's operands
// The ring lies at the bottom of LDS and the epilogue staging right above it: every destination of a global-to-LDS load
// stays below 128 KB (a variant that put such destinations higher ended in a memory fault whose cause was never found).
static_assert(kRingStages * kRingStageBytes + kRingWaves * kRingAuxBytes <= 128 * 1024,
              "global-to-LDS destinations must stay below 128 KB");
constexpr int kRingLoadsPerWave = kRingRows / 16 / kRingWaves;  // wave-wide 1 KB loads per stage and wavefront

// Operand fragments of one half-step: 4 query blocks and 2 base blocks of 32 rows, 16 bytes per lane.
template <typename V>
struct RingFrag {
    V a[4], b[2];
};

// The fragment reads and the waits for them are written as inline assembly: the compiler would wait
// for ALL outstanding LDS reads before the first MFMA of a half-step (it merges the counter states
// of the loop's paths conservatively), which serialises the reads of the next half-step with the
// MFMAs of the current one.  LDS reads complete in order, so "at most 6 outstanding" after issuing
// the 6 reads of the next fragment set means the previous set has arrived.  Scalar loads share the
// counter but can only make the wait stricter than needed, never weaker.
// a_addr / b_addr: LDS byte address of this lane's chunk in the first query / base block of the stage.
template <typename V>
__device__ __forceinline__ void ring_read_frag(uint32_t a_addr, uint32_t b_addr, RingFrag<V> &f)
{
    asm volatile("ds_read_b128 %0, %1" : "=v"(f.a[0]) : "v"(a_addr));
    asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(f.a[1]) : "v"(a_addr));
    asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(f.a[2]) : "v"(a_addr));
    asm volatile("ds_read_b128 %0, %1 offset:6144" : "=v"(f.a[3]) : "v"(a_addr));
    asm volatile("ds_read_b128 %0, %1" : "=v"(f.b[0]) : "v"(b_addr));
    asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(f.b[1]) : "v"(b_addr));
}
// Waits until at most N LDS operations are outstanding; the fragment registers pass through the
// statement so that no use of them can be scheduled ahead of it.
template <int N, typename V>
__device__ __forceinline__ void ring_wait_frag(RingFrag<V> &f)
{
    asm volatile("s_waitcnt lgkmcnt(%6)"
                 : "+v"(f.a[0]), "+v"(f.a[1]), "+v"(f.a[2]), "+v"(f.a[3]), "+v"(f.b[0]), "+v"(f.b[1])
                 : "n"(N));
}

// bf16 operands, fp32 accumulation (v_mfma_f32_32x32x16_bf16): same data movement as int8.
struct Bf16Traits {
    using T = uint16_t;
    using S = float;
    using Acc = v16f;
    using Frag = RingFrag<bf16x8>;
    static constexpr int kElemsPerStep = 32;
    static __device__ __forceinline__ int chunk(int hs, int half) { return hs * 2 + half; }
    template <bool SWAP, bool ZERO>
    static __device__ __forceinline__ void mma(const Frag &f, Acc (&acc)[4][2])
    {
#pragma unroll
        for (int ra = 0; ra < 4; ra++) {
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const Acc c0 = ZERO ? Acc{} : acc[ra][rb];
                acc[ra][rb] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.b[rb], f.a[ra], c0, 0, 0, 0)
                                   : __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[ra], f.b[rb], c0, 0, 0, 0);
            }
        }
    }
};

struct F32Traits {
    using T = float;
    using S = float;
    using Acc = v16f;
    using Frag = RingFrag<v4f>;
    static constexpr int kElemsPerStep = 16;
    // one K-step = 16 floats; a lane half owns 8 of them (two 16-byte chunks), one chunk per half-step,
    // fed to 4 consecutive 32x32x2 MFMAs
    static __device__ __forceinline__ int chunk(int hs, int half) { return half * 2 + hs; }
    template <bool SWAP, bool ZERO>
    static __device__ __forceinline__ void mma(const Frag &f, Acc (&acc)[4][2])
    {
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const float av = f.a[ra][t], bv = f.b[rb][t];
                    const Acc c0 = (ZERO && t == 0) ? Acc{} : acc[ra][rb];
                    acc[ra][rb] = SWAP ? __builtin_amdgcn_mfma_f32_32x32x2f32(bv, av, c0, 0, 0, 0)
                                       : __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, c0, 0, 0, 0);
                }
            }
        }
    }
};

// s_waitcnt immediate that waits until at most n vector-memory operations are outstanding and
// leaves the other counters alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
__host__ __device__ constexpr int ring_vmcnt(int n)
{
    return 0x0f70 | ((n > 63 ? 63 : n) & 15) | (((n > 63 ? 63 : n) >> 4) << 14);
}

// MODE 0: the scores are stored.  MODE 1: scores at or below the row's bound are appended as keys, one
// atomic per key.  MODE 2 (fp32 scores): runs of four consecutive columns whose smallest score is at or below
// the row's bound are appended as 32-byte records {four scores, first column, unused x 3}; a lane counts its
// passing runs of a query row first and reserves their places with ONE atomic, so a tile costs a wave four
// atomic round trips whatever the admission rate.  MODE 3 (fp32 scores): nothing but group minima leave the
// kernel: out[row * ldo + 8 * base tile + 2 * (wave column) + lane half] = the smallest score of the row among
// that lane's 32 columns of the tile (+inf where it has none).
template <typename Tr, int MODE>
__global__ __launch_bounds__(kRingWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void score_ring_kernel(
    const typename Tr::T *__restrict__ Q, int64_t nq, const typename Tr::T *__restrict__ B, int64_t nb, int d,
    const typename Tr::S *__restrict__ qn, const typename Tr::S *__restrict__ bn, int metric,
    typename Tr::S *__restrict__ out, int64_t ldo, int tiles_m, int tiles_n, ScoreFilter<typename Tr::S> flt)
{
    using T = typename Tr::T;
    using S = typename Tr::S;
    constexpr bool FILTER = MODE != 0, DUMP = MODE == 2, MINIMA = MODE == 3;
    static_assert(std::is_same<S, float>::value, "floating-point scores");
    extern __shared__ __align__(16) unsigned char ring[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 2, wc = wave & 3;
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

    // Sources of the tile whose K-steps are being issued.  Waves 0..3 load the query rows, waves 4..7
    // the base rows: a wave-uniform tile base plus a 32-bit per-lane byte offset per load (recomputed
    // once per tile; rows past the end of the operand re-read its last row); a K-step then only
    // advances the uniform base by ks * 64 bytes.
    const bool loads_q = wave < kRingTM / 16 / kRingLoadsPerWave;
    const unsigned char *tile_base = nullptr;
    uint32_t src_off[kRingLoadsPerWave];
    auto set_sources = [&](int it) {
        int64_t tm, tn;
        item_tile(it, tm, tn);
        const int64_t row0 = loads_q ? tm * kRingTM : tn * kRingTN;
        const int64_t last = (loads_q ? nq : nb) - 1 - row0;     // >= 0: the tile exists
        const int limit = (int)(last < kRingTM - 1 ? last : kRingTM - 1);
        tile_base = (loads_q ? Qb : Bb) + row0 * row_bytes;
#pragma unroll
        for (int j = 0; j < kRingLoadsPerWave; j++) {
            const int rg = wave * kRingLoadsPerWave + j;          // group of 16 stage rows
            const int row = rg * 16 + (lane >> 2);                // stage row: 0..255 queries, 256..511 base
            const int chunk = (lane & 3) ^ ((row >> 2) & 3);
            const int local = row & (kRingTM - 1);                // row inside the operand tile
            src_off[j] = (uint32_t)(local < limit ? local : limit) * (uint32_t)row_bytes + (uint32_t)chunk * 16u;
        }
    };
    // issue the loads of one K-step (step ks of the current issue tile) into ring buffer `slot`
    auto issue = [&](int ks, int slot) {
        unsigned char *stage = ring + slot * kRingStageBytes;
        const unsigned char *base = tile_base + ks * 64;
#pragma unroll
        for (int j = 0; j < kRingLoadsPerWave; j++) {
            const int rg = wave * kRingLoadsPerWave + j;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(base + src_off[j]),
                                             (__attribute__((address_space(3))) void *)(stage + rg * 1024), 16, 0, 0);
        }
    };

    typename Tr::Acc acc[4][2];   // written from zero by the first half-step of every tile

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
    // The two wavefronts of a SIMD (waves w and w + 4) do their per-step bookkeeping (address updates
    // and load issue: a few hundred cycles without an MFMA) at different points between the
    // once-per-step barriers, so that one wave's bookkeeping coincides with the other's MFMAs:
    // "early" waves (0..3) right after the barrier, "late" waves (4..7) after the second half-step.
    const bool late = wave >= 4;
    while (issued < kRingStages && issued < total) {
        issue_next();
    }
    int c_it = 0, c_ks = 0, c_slot = 0;
    bool stored = false;  // the previous K-step ended with an epilogue that issued stores

    // Filtered launches stage what the epilogue of a tile needs -- the base norms of the wave's 64
    // columns and the bounds (and norms) of its 128 query rows -- in a small per-wave LDS area, with
    // the same global->LDS loads as the ring and one K-step ahead, so the epilogue never waits for
    // memory and the main loop carries no registers for it.  The s_waitcnt immediates below count
    // these loads (kPrefetchLoads per wave).
    //   aux +   0: 64 base norms      (lanes 0..15, 16 bytes each)
    //   aux + 256: 128 tau or thr     (lanes 16..47)
    //   aux + 768: 128 query norms    (lanes 0..31 of a second load)
    constexpr int kPrefetchLoads = 2;
    unsigned char *aux = ring + kRingStages * kRingStageBytes + wave * kRingAuxBytes;
    const S *bound = flt.tau;
    const bool prefetch = FILTER && nk >= 2 && nb % 4 == 0 && nq % 4 == 0 && bn != nullptr && qn != nullptr &&
                          bound != nullptr && reinterpret_cast<uintptr_t>(bn) % 16 == 0 &&
                          reinterpret_cast<uintptr_t>(qn) % 16 == 0 && reinterpret_cast<uintptr_t>(bound) % 16 == 0;
    bool fetched = false;   // the staging loads were issued during the previous K-step
    auto fetch_epilogue_operands = [&](int it) {
        int64_t tm, tn;
        item_tile(it, tm, tn);
        const int64_t i0 = tm * kRingTM, j0 = tn * kRingTN;
        asm volatile("" ::: "memory");
        // (the lane number is made opaque here so that nothing derived from it in this once-per-tile
        // code is kept in registers across the main loop)
        int lane = tid & 63;
        asm volatile("" : "+v"(lane));
        // groups of four values; a group that starts past the end of its array reads the array's
        // first group instead (its scores are rejected by index in the epilogue)
        if (lane < 48) {
            const bool is_bn = lane < 16;
            const int group = is_bn ? lane : lane - 16;
            const int64_t first = is_bn ? j0 + wc * 64 : i0 + wr * 128;
            const int64_t left = ((is_bn ? nb : nq) - first) >> 2;      // whole groups from `first` on
            const S *arr = is_bn ? bn : bound;
            const S *p = group < left ? arr + first + group * 4 : arr;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                             (__attribute__((address_space(3))) void *)aux, 16, 0, 0);
        }
        if (lane < 32) {
            const int64_t first = i0 + wr * 128;
            const S *p = lane < ((nq - first) >> 2) ? qn + first + lane * 4 : qn;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)p,
                                             (__attribute__((address_space(3))) void *)(aux + 768), 16, 0, 0);
        }
        asm volatile("" ::: "memory");
    };

    // K-step 0 must have landed before its first fragments are read
    if (issued >= 3) {
        __builtin_amdgcn_s_waitcnt(ring_vmcnt(2 * kRingLoadsPerWave));
    } else if (issued == 2) {
        __builtin_amdgcn_s_waitcnt(ring_vmcnt(kRingLoadsPerWave));
    } else {
        __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
    }
    __builtin_amdgcn_s_barrier();
    // LDS addresses of this lane's fragment chunks: row blocks are 2048 bytes apart (immediate
    // offsets); the swizzle term (row >> 2) & 3 only depends on the lane
    const uint32_t ring_base = (uint32_t)reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)ring);
    const int swz = (l32 >> 2) & 3;
    const uint32_t a_row = ring_base + (uint32_t)(wr * 128 + l32) * 64, b_row = ring_base + (uint32_t)(kRingTM + wc * 64 + l32) * 64;
    const uint32_t coff0 = (uint32_t)((Tr::chunk(0, half) ^ swz) << 4), coff1 = (uint32_t)((Tr::chunk(1, half) ^ swz) << 4);
    typename Tr::Frag fa, fb;
    ring_read_frag(a_row + coff0, b_row + coff0, fa);

    for (int g = 0; g < total; g++) {
        const uint32_t stage_off = (uint32_t)(c_slot * kRingStageBytes);
        const int next_slot = c_slot + 1 == kRingStages ? 0 : c_slot + 1;
        bool issued_now = false;
        // the wait a wave does before barrier g: K-step g + 1 (its own part) must have landed.  vmcnt
        // counts loads and stores in issue order; younger than the loads of K-step g + 1 are the loads
        // of K-step g + 2 and the staging loads of a filtered epilogue, when those were issued.  A
        // storing epilogue does this wait itself, before it issues its stores.
        auto wait_next_step = [&]() {
            if (g + 2 >= total) {
                __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
            } else if (!FILTER && stored) {
            } else if (FILTER && fetched) {
                __builtin_amdgcn_s_waitcnt(ring_vmcnt(kRingLoadsPerWave + kPrefetchLoads));
            } else {
                __builtin_amdgcn_s_waitcnt(ring_vmcnt(kRingLoadsPerWave));
            }
        };
        auto issue_and_fetch = [&]() {
            if (issued < total) {
                issue_next();  // into the buffer of K-step g
                issued_now = true;
            }
            if (FILTER && prefetch && c_ks == nk - 2) {
                fetch_epilogue_operands(c_it);
                fetched = true;
            } else {
                fetched = false;
            }
        };
        // ---- first half-step: its fragments (fa) were read during the previous half-step
        ring_read_frag(a_row + stage_off + coff1, b_row + stage_off + coff1, fb);
        ring_wait_frag<6>(fa);
        if (c_ks == 0) {
            Tr::template mma<FILTER, true>(fa, acc);
        } else {
            Tr::template mma<FILTER, false>(fa, acc);
        }
        // ---- between the half-steps: barrier g.  Before it K-step g + 1 (this wave's part) must have
        // landed and this wave must be done reading the buffer of K-step g (its second fragments are
        // in registers once lgkmcnt is 0); after it K-step g + 3 may overwrite that buffer.
        ring_wait_frag<0>(fb);
        if (g + 1 < total) {
            wait_next_step();
            __builtin_amdgcn_s_barrier();
            if (!late) {
                issue_and_fetch();
            }
            const uint32_t next_off = (uint32_t)(next_slot * kRingStageBytes);
            ring_read_frag(a_row + next_off + coff0, b_row + next_off + coff0, fa);
        }
        stored = false;
        // ---- second half-step
        Tr::template mma<FILTER, false>(fb, acc);
        const bool last_step = c_ks == nk - 1;
        const int done_it = c_it;
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
            // lane-derived values of this once-per-tile code must not occupy registers in the main loop
            int lane = tid & 63;
            asm volatile("" : "+v"(lane));
            const int half = lane >> 5, l32 = lane & 31;
            // The epilogue's operands come out of the wave's staging area: put there one K-step ahead
            // by fetch_epilogue_operands(), or (shapes the staging loads do not serve) filled here.
            if (prefetch) {
                // the staging loads are older than the K-step loads issued during this K-step
                if (issued_now) {
                    __builtin_amdgcn_s_waitcnt(ring_vmcnt(kRingLoadsPerWave));
                } else {
                    __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
                }
                asm volatile("" ::: "memory");
            } else {
                const int64_t col = j0 + wc * 64 + lane;
                reinterpret_cast<S *>(aux)[lane] = (metric == kMetricL2 && col < nb) ? bn[col] : (S)0;
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const int64_t row = i0 + wr * 128 + t * 64 + lane;
                    const bool ok = row < nq;
                    reinterpret_cast<S *>(aux + 256)[t * 64 + lane] = ok ? bound[row] : (S)0;
                    reinterpret_cast<S *>(aux + 768)[t * 64 + lane] = (ok && metric == kMetricL2) ? qn[row] : (S)0;
                }
            }
            wave_lds_fence();
            if constexpr (MINIMA) {
#pragma unroll
                for (int ra = 0; ra < 4; ra++) {
                    asm volatile("" ::: "memory");   // one query block at a time keeps register pressure low
                    const int64_t row = i0 + (wr * 128 + ra * 32 + l32);
                    const float rowv = *reinterpret_cast<const float *>(aux + 768 + (ra * 32 + l32) * 4);
                    int cb = wc * 64 + 4 * half;
                    asm volatile("" : "+v"(cb));
                    float best = __builtin_inff();
#pragma unroll
                    for (int rb = 0; rb < 2; rb++) {
#pragma unroll
                        for (int rq = 0; rq < 4; rq++) {
                            const uint4 u = *reinterpret_cast<const uint4 *>(aux + (rb * 32 + 8 * rq + 4 * half) * 4);
                            const float bnq[4] = {__builtin_bit_cast(float, u.x), __builtin_bit_cast(float, u.y),
                                                  __builtin_bit_cast(float, u.z), __builtin_bit_cast(float, u.w)};
                            float m = __builtin_inff();
#pragma unroll
                            for (int t = 0; t < 4; t++) {
                                const float g = acc[ra][rb][rq * 4 + t];
                                float w;
                                if (metric == kMetricL2) {
                                    w = __fadd_rn(rowv, bnq[t]);
                                    w = __fsub_rn(w, g);
                                    w = __fsub_rn(w, g);
                                } else {
                                    w = -g;
                                }
                                m = fminf(m, w);
                            }
                            // columns past the end of the base re-read its last row: they count for nothing
                            // (the base has a multiple of four rows, so a run of four is inside or outside)
                            best = j0 + cb + rb * 32 + 8 * rq < nb ? fminf(best, m) : best;
                        }
                    }
                    if (row < nq) {
                        out[row * ldo + (tn * 8 + wc * 2 + half)] = best;
                    }
                }
            } else if constexpr (DUMP) {
                unsigned char *records = reinterpret_cast<unsigned char *>(flt.cand);
#pragma unroll
                for (int ra = 0; ra < 4; ra++) {
                    asm volatile("" ::: "memory");   // one query block at a time keeps register pressure low
                    const int64_t row = i0 + (wr * 128 + ra * 32 + l32);
                    const bool row_ok = row < nq;
                    const float tauv = *reinterpret_cast<const float *>(aux + 256 + (ra * 32 + l32) * 4);
                    const float rowv = *reinterpret_cast<const float *>(aux + 768 + (ra * 32 + l32) * 4);
                    float v[2][16];
                    int npass = 0;
                    int cb = wc * 64 + 4 * half;   // opaque: no column offsets live across the main loop
                    asm volatile("" : "+v"(cb));
#pragma unroll
                    for (int rb = 0; rb < 2; rb++) {
#pragma unroll
                        for (int rq = 0; rq < 4; rq++) {
                            const uint4 u = *reinterpret_cast<const uint4 *>(aux + (rb * 32 + 8 * rq + 4 * half) * 4);
                            const float bnq[4] = {__builtin_bit_cast(float, u.x), __builtin_bit_cast(float, u.y),
                                                  __builtin_bit_cast(float, u.z), __builtin_bit_cast(float, u.w)};
#pragma unroll
                            for (int t = 0; t < 4; t++) {
                                const float g = acc[ra][rb][rq * 4 + t];
                                float w;
                                if (metric == kMetricL2) {
                                    w = __fadd_rn(rowv, bnq[t]);
                                    w = __fsub_rn(w, g);
                                    w = __fsub_rn(w, g);
                                } else {
                                    w = -g;
                                }
                                v[rb][rq * 4 + t] = w;
                            }
                            const float m = fminf(fminf(v[rb][rq * 4], v[rb][rq * 4 + 1]),
                                                  fminf(v[rb][rq * 4 + 2], v[rb][rq * 4 + 3]));
                            // columns past the end of the base re-read its last row: never admitted
                            const bool pass = row_ok && m <= tauv && j0 + cb + rb * 32 + 8 * rq < nb;
                            npass += pass ? 1 : 0;
                        }
                    }
                    int pos = 0;
                    if (npass > 0) {
                        pos = atomicAdd(&flt.cnt[row], npass);
                    }
                    unsigned char *rec = records + ((int64_t)row * flt.cap + pos) * 32;
#pragma unroll
                    for (int rb = 0; rb < 2; rb++) {
#pragma unroll
                        for (int rq = 0; rq < 4; rq++) {
                            const float m = fminf(fminf(v[rb][rq * 4], v[rb][rq * 4 + 1]),
                                                  fminf(v[rb][rq * 4 + 2], v[rb][rq * 4 + 3]));
                            const int64_t col = j0 + cb + rb * 32 + 8 * rq;
                            if (row_ok && m <= tauv && col < nb) {
                                if (pos < flt.cap) {
                                    *reinterpret_cast<float4 *>(rec) = make_float4(v[rb][rq * 4], v[rb][rq * 4 + 1],
                                                                                   v[rb][rq * 4 + 2], v[rb][rq * 4 + 3]);
                                    *reinterpret_cast<uint32_t *>(rec + 16) = (uint32_t)(col + flt.col_base);
                                }
                                pos++;
                                rec += 32;
                            }
                        }
                    }
                }
            } else {
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                asm volatile("" ::: "memory");   // one query block at a time keeps register pressure low
                const int64_t row = i0 + (wr * 128 + ra * 32 + l32);
                const bool row_ok = row < nq;
                const S tauv = *reinterpret_cast<const S *>(aux + 256 + (ra * 32 + l32) * 4);
                const S rowv = *reinterpret_cast<const S *>(aux + 768 + (ra * 32 + l32) * 4);
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    // all 16 scores of the block first, then ONE test of their minimum against the
                    // lane's bound: admissions are rare, so the per-score path almost never runs
                    S v[16];
                    S best = ScoreOps<S>::worst();
                    S bnq[4][4];   // the base norms of this lane's 16 columns of the block
#pragma unroll
                    for (int rq = 0; rq < 4; rq++) {
                        const uint4 u = *reinterpret_cast<const uint4 *>(aux + (rb * 32 + 8 * rq + 4 * half) * 4);
                        bnq[rq][0] = __builtin_bit_cast(S, u.x);
                        bnq[rq][1] = __builtin_bit_cast(S, u.y);
                        bnq[rq][2] = __builtin_bit_cast(S, u.z);
                        bnq[rq][3] = __builtin_bit_cast(S, u.w);
                    }
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const S bnv = bnq[r >> 2][r & 3];
                        const float g = acc[ra][rb][r];
                        if (metric == kMetricL2) {
                            float w = __fadd_rn(rowv, bnv);
                            w = __fsub_rn(w, g);
                            v[r] = __fsub_rn(w, g);
                        } else {
                            v[r] = -g;
                        }
                        best = v[r] < best ? v[r] : best;
                    }
                    const S lane_bound = tauv;
                    if (__ballot(row_ok && best <= lane_bound)) {
                        // opaque to the optimiser here, or it keeps all 32 column offsets of this rare
                        // path in registers across the whole main loop
                        int cb = wc * 64 + rb * 32 + 4 * half;
                        asm volatile("" : "+v"(cb));
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int64_t col = j0 + cb + 8 * (r >> 2) + (r & 3);
                            if (row_ok && v[r] <= lane_bound && col < nb) {
                                const int pos = atomicAdd(&flt.cnt[row], 1);
                                if (pos < flt.cap) {
                                    flt.cand[row * flt.cap + pos] = make_key(v[r], (uint32_t)(col + flt.col_base));
                                }
                            }
                        }
                    }
                }
            }
            }   // !DUMP
        }
        if (!FILTER && last_step) {
            // The stores below queue up behind the loads in flight, and how many of them a wave issues
            // depends on the tile's position: the wait for the next K-step that the coming barrier
            // needs happens here, while the loads are still the youngest operations.
            if (issued_now) {
                __builtin_amdgcn_s_waitcnt(ring_vmcnt(kRingLoadsPerWave));
            } else {
                __builtin_amdgcn_s_waitcnt(ring_vmcnt(0));
            }
            stored = true;
            int64_t tm, tn;
            item_tile(done_it, tm, tn);
            const int64_t i0 = tm * kRingTM, j0 = tn * kRingTN;
            S bnv[2];
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
                const int64_t col = j0 + wc * 64 + rb * 32 + l32;
                bnv[rb] = (col < nb && metric == kMetricL2) ? bn[col] : (S)0;
            }
#pragma unroll
            for (int ra = 0; ra < 4; ra++) {
                // one 32-row block at a time keeps the per-row operands of only 16 rows live
                asm volatile("" ::: "memory");
                S rowv[16];   // |q|^2
                S tauv[16];   // FILTER: tau
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int64_t row = i0 + wr * 128 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    rowv[r] = (row < nq && metric == kMetricL2) ? qn[row] : (S)0;
                    tauv[r] = (FILTER && row < nq) ? flt.tau[row] : (S)(-__builtin_inff());
                }
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    const int64_t col = j0 + wc * 64 + rb * 32 + l32;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int64_t row = i0 + wr * 128 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                        S v;
                        const float g = acc[ra][rb][r];
                        if (metric == kMetricL2) {
                            v = __fadd_rn(rowv[r], bnv[rb]);
                            v = __fsub_rn(v, g);
                            v = __fsub_rn(v, g);
                        } else {
                            v = -g;
                        }
                        const bool admit = v <= tauv[r];
                        if (FILTER) {
                            if (admit && col < nb) {
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
        if (late && g + 1 < total) {
            issue_and_fetch();
        }
        c_slot = next_slot;
        if (++c_ks == nk) {
            c_ks = 0;
            c_it++;
        }
    }
}

template <typename Tr, int MODE>
void launch_ring_mode(const typename Tr::T *Q, int64_t nq, const typename Tr::T *B, int64_t nb, int d,
                      const typename Tr::S *qn, const typename Tr::S *bn, int metric, typename Tr::S *out, int64_t ldo,
                      ScoreFilter<typename Tr::S> flt, int64_t rt_m, int64_t rt_n, unsigned grid, hipStream_t s)
{
    const size_t smem = (size_t)kRingStages * kRingStageBytes + (MODE != 0 ? kRingWaves * kRingAuxBytes : 0);
    auto kern = score_ring_kernel<Tr, MODE>;
    require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kRingWaves * 64), smem, s, Q, nq, B, nb, d, qn, bn, metric, out, ldo,
                       (int)rt_m, (int)rt_n, flt);
}

// mode: 0 = store the scores, 1 = append admitted keys, 2 = append admitted runs of four as records
// (floating-point scores only)
template <typename Tr>
bool launch_ring(const typename Tr::T *Q, int64_t nq, const typename Tr::T *B, int64_t nb, int d,
                 const typename Tr::S *qn, const typename Tr::S *bn, int metric, typename Tr::S *out, int64_t ldo,
                 int mode, ScoreFilter<typename Tr::S> flt, hipStream_t s)
{
    if (d % Tr::kElemsPerStep != 0 || nb < 8 * kRingTN || reinterpret_cast<uintptr_t>(Q) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(B) % 16 != 0) {
        return false;
    }
    const int64_t rt_m = (nq + kRingTM - 1) / kRingTM, rt_n = (nb + kRingTN - 1) / kRingTN;
    if (rt_m * rt_n >= ((int64_t)1 << 31) || rt_m * ((rt_n + 7) / 8) * (d / Tr::kElemsPerStep) >= ((int64_t)1 << 30)) {
        return false;
    }
    static std::atomic<int> known{0};
    int cus = known.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        IXA_HIP(hipGetDevice(&dev));
        IXA_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        known.store(cus, std::memory_order_relaxed);
    }
    const unsigned grid = (unsigned)((cus + 7) / 8 * 8);   // one persistent workgroup per CU
    if (mode == 2 || mode == 3) {
        if constexpr (sizeof(typename Tr::T) == 2) {
            if (mode == 2) {
                launch_ring_mode<Tr, 2>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, flt, rt_m, rt_n, grid, s);
            } else {
                launch_ring_mode<Tr, 3>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, flt, rt_m, rt_n, grid, s);
            }
            return true;
        }
        return false;
    }
    if (mode == 1) {
        launch_ring_mode<Tr, 1>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, flt, rt_m, rt_n, grid, s);
    } else {
        launch_ring_mode<Tr, 0>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, flt, rt_m, rt_n, grid, s);
    }
    return true;
}

}  // namespace

bool launch_score_ring_bf16(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                            const float *bn, int metric, float *out, int64_t ldo, bool filter, ScoreFilter<float> flt,
                            hipStream_t s)
{
    return launch_ring<Bf16Traits>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, filter ? 1 : 0, flt, s);
}

bool launch_score_ring_bf16_minima(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                                   const float *bn, int metric, float *out, int64_t ldo, hipStream_t s)
{
    ScoreFilter<float> flt{};
    flt.tau = qn;   // the epilogue's operand staging wants a bound array; this mode reads none of it
    return launch_ring<Bf16Traits>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, 3, flt, s);
}

bool launch_score_ring_bf16_records(const uint16_t *Q, int64_t nq, const uint16_t *B, int64_t nb, int d, const float *qn,
                                    const float *bn, int metric, ScoreFilter<float> flt, hipStream_t s)
{
    return launch_ring<Bf16Traits>(Q, nq, B, nb, d, qn, bn, metric, nullptr, 0, 2, flt, s);
}

// Appends a query to the list flag[1 + flag[0]++] unless, for that query, no centroid outside its approximate candidate list can beat
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
        flag[1 + atomicAdd(flag, 1)] = (int)i;   // the list of queries that need another plan
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
    return launch_ring<F32Traits>(Q, nq, B, nb, d, qn, bn, metric, out, ldo, filter ? 1 : 0, flt, s);
}

}  // namespace ixa
