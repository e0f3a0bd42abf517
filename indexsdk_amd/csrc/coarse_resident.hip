// Coarse-stage scores with the query tile resident in LDS: the bf16 x 3 query x centroid product of the sampled-bound
// plan (stream_select.h) in the structure of the int8 Flat kernel (flat_i8.hip).
//
//   * a persistent workgroup of 8 wavefronts copies a tile of QT = 32 RA split queries ([hi | hi | lo] rows of d3 bf16,
//     score_ring.hip) into LDS once, as [16-byte chunk of K][query][16 B], and walks 256-row tiles of the split
//     centroids with it; the centroids are stored in matrix-core order (blocks of 32 rows as [chunk][row][16 B],
//     flat_i8.h) once, when the quantizer is set, so a wavefront's operand fragment of a K-step is 1 KB of contiguous
//     memory that goes straight into registers: no LDS ring, no workgroup barrier in the main loop;
//   * wavefront w owns centroids 32 w .. 32 w + 31 of the tile and all queries: per K-step one global_load_dwordx4, RA
//     ds_read_b128 and RA v_mfma_f32_32x32x16_bf16;
//   * the centroid fragment is the first matrix operand, so a lane owns ONE query per accumulator block and 16
//     centroids (four runs of four consecutive ones).
// Two epilogues, the same two the ring kernel has for this plan:
//   MINIMA   out[row * ldo + 8 tile + wave] = the smallest score of the row among the 32 centroids of that wavefront
//            (scores in the ring kernel's arithmetic: (|q|^2 + |c|^2) - g - g, or -g for inner product);
//   RECORDS  every run of four centroids that holds a score at or below the row's bound is appended to the row's
//            records as {the four DOT PRODUCTS g, first centroid}: the test is made on u = g - |c|^2 / 2 (one fused
//            multiply-add per score) against a per-query value that lies below (|q|^2 - tau) / 2 by more than the
//            roundings of both forms can differ, so no run with a score <= tau is missed; the fold that reads the
//            records turns g into scores (launch_fold_* with raw = true).  Records are compacted over the lanes into
//            a per-wavefront queue in LDS and leave 64 at a time (one atomic and two stores per lane).
#include <cmath>

#include "coarse.h"
#include "flat_i8.h"
#include "resident_tile.h"
#include "topk.h"

namespace ixa {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kQueueRecords = 128;   // per wavefront, 32 bytes each; flushed when fewer than 64 places are left
enum { kMinima = 0, kRecords = 1 };

template <int NHS, int PF, int RA, int MODE>
__global__ __launch_bounds__(kWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void resident_bf16_kernel(
    const uint16_t *__restrict__ Qs, int64_t nq, const uint16_t *__restrict__ Bt, const float *__restrict__ cnp, int64_t nb,
    const float *__restrict__ qn, const float *__restrict__ test, int metric, float *__restrict__ out, int64_t ldo,
    ScoreFilter<float> flt, int tiles_m, int ntiles, int seg_tiles, int own_resident)
{
    constexpr int D = NHS * 32, QT = RA * 32;   // bytes of a split row, queries of a tile
    constexpr int kStepLds = QT * 32;           // LDS bytes of one K-step: two chunks of QT x 16 bytes
    static_assert(NHS % PF == 0, "shape");
    extern __shared__ __align__(16) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, l32 = lane & 31;
    const int xcd = blockIdx.x & 7, wi = blockIdx.x >> 3, wpx = gridDim.x >> 3;
    const ResidentItems sched(tiles_m, ntiles, seg_tiles, xcd, wpx, own_resident != 0);
    const int S = sched.S;
    const int first_item = sched.next(wi);
    if (first_item < 0) {
        return;
    }
    const uint32_t lds_base = (uint32_t)reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)lds);
    // + step * kStepLds + block * 512: the offset field of a read holds 16 bits, so there is a base every 32 KB and
    // the offsets of a group of RA reads stay below 32768 + 512 RA
    constexpr int kBases = (NHS * kStepLds + 32767) / 32768;
    uint32_t a_lane[kBases];
#pragma unroll
    for (int i = 0; i < kBases; i++) {
        a_lane[i] = lds_base + (uint32_t)(half * (QT * 16) + l32 * 16) + 32768u * i;
    }
    float *perq = reinterpret_cast<float *>(lds + QT * D);   // per query: the test value (RECORDS) or |q|^2 (MINIMA)
    const unsigned char *Bb = reinterpret_cast<const unsigned char *>(Bt);
    const unsigned char *Qb = reinterpret_cast<const unsigned char *>(Qs);
    auto block_row0 = [&](int j) { return sched.streamed_tile(j) * kI8TileRows + wave * 32; };
    auto block_ptr = [&](int j) { return Bb + block_row0(j) * (int64_t)D + lane * 16; };

    v16f acc[RA];
    bf16x8 breg[PF];
    v4f cnv[4];   // |c|^2 of the lane's 16 centroids of the current tile
    // RECORDS: the wavefront's queue of records on their way out, 32 bytes each: {four dot products | first centroid,
    // query row, -, -}
    uint4 *queue = reinterpret_cast<uint4 *>(lds + QT * D + QT * 4) + wave * (2 * kQueueRecords);
    int qcount = 0;   // wave-uniform
    auto flush_queue = [&]() {
        wave_lds_fence();
        unsigned char *records = reinterpret_cast<unsigned char *>(flt.cand);
        for (int i0 = 0; i0 < qcount; i0 += 64) {
            if (i0 + lane < qcount) {
                const uint4 sc = queue[2 * (i0 + lane)], id = queue[2 * (i0 + lane) + 1];
                const int p = atomicAdd(&flt.cnt[id.y], 1);
                if (p < flt.cap) {
                    unsigned char *rec = records + ((int64_t)id.y * flt.cap + p) * 32;
                    *reinterpret_cast<uint4 *>(rec) = sc;
                    *reinterpret_cast<uint32_t *>(rec + 16) = id.x;
                }
            }
        }
        wave_lds_fence();
        qcount = 0;
    };
    int cur_tm = -1;
    int it_t = first_item;
    int tm, j, jend;
    sched.range(it_t, tm, j, jend);
    const unsigned char *cur = block_ptr(j);
#pragma unroll
    for (int p = 0; p < PF; p++) {
        breg[p] = *reinterpret_cast<const bf16x8 *>(cur + p * 1024);
    }
    bool staggered = false;
    while (true) {
        if (tm != cur_tm) {
            if (cur_tm >= 0) {
                __syncthreads();
            }
            load_resident_tile<QT, D, kWaves * 64>(lds, Qb, (int64_t)tm * QT, nq, tid);
            if (tid < QT) {
                const int64_t row = (int64_t)tm * QT + tid;
                if constexpr (MODE == kRecords) {
                    perq[tid] = row < nq ? test[row] : __builtin_inff();   // rows past the end admit nothing
                } else {
                    perq[tid] = (row < nq && metric == kMetricL2) ? qn[row] : 0.f;
                }
            }
            cur_tm = tm;
            __syncthreads();
            // the second wavefront of every SIMD starts half a tile late, so that each one's epilogue runs under the
            // other's matrix instructions
            if (!staggered && wave >= kWaves / 2) {
                constexpr int kHalfTile = NHS * RA / 2;
                __builtin_amdgcn_s_sleep(kHalfTile < 127 ? kHalfTile : 127);
            }
            staggered = true;
        }
        int n_it = it_t, n_tm = tm, n_j = j + S, n_jend = jend;
        bool has_next = true;
        if (n_j >= jend) {
            n_it = sched.next(it_t + wpx);
            if (n_it >= 0) {
                sched.range(n_it, n_tm, n_j, n_jend);
            } else {
                has_next = false;
                n_it = it_t;
                n_j = j;
            }
        }
        const unsigned char *nxt = block_ptr(n_j);
        // the norms of this tile's centroids: wanted by the epilogue only, so their loads have the whole tile to land;
        // issued before the tile's fragment loads so that waiting for them never drains those
        {
            const float *cp = cnp + block_row0(j) + 4 * half;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                cnv[g] = *reinterpret_cast<const v4f *>(cp + 8 * g);
            }
            asm volatile("" ::: "memory");
        }
        bf16x8 fa[2][RA];
        lds_read_group<RA, 0>(a_lane[0], fa[0]);
        static_for<0, NHS>([&](auto hc) {
            constexpr int hs = decltype(hc)::value;
            if constexpr (hs + 1 < NHS) {
                constexpr int off = (hs + 1) * kStepLds;
                lds_read_group<RA, off % 32768>(a_lane[off / 32768], fa[(hs + 1) & 1]);
                lds_wait_group<RA, RA>(fa[hs & 1]);
            } else {
                lds_wait_group<RA, 0>(fa[hs & 1]);
            }
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                if constexpr (hs == 0) {
                    acc[ra] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(breg[0], fa[0][ra], v16f{}, 0, 0, 0);
                } else {
                    acc[ra] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(breg[hs % PF], fa[hs & 1][ra], acc[ra], 0, 0, 0);
                }
            }
            if constexpr (hs + PF < NHS) {
                breg[hs % PF] = *reinterpret_cast<const bf16x8 *>(cur + (hs + PF) * 1024);
            } else {
                breg[hs % PF] = *reinterpret_cast<const bf16x8 *>(nxt + (hs + PF - NHS) * 1024);
            }
            asm volatile("" ::: "memory");
        });
        // a lane owns query (block ra, l32) and centroids col0 + 8 g + t of the wave's block (g: run, t: 0..3)
        const int64_t col0 = block_row0(j) + 4 * half;
        if constexpr (MODE == kMinima) {
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                const float rowv = perq[ra * 32 + l32];
                float best = __builtin_inff();
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float g = acc[ra][r];
                    float v;
                    if (metric == kMetricL2) {
                        v = __fadd_rn(rowv, cnv[r >> 2][r & 3]);
                        v = __fsub_rn(v, g);
                        v = __fsub_rn(v, g);
                    } else {
                        v = -g;
                    }
                    best = fminf(best, v);
                }
                best = fminf(best, __shfl_xor(best, 32));   // both halves: the wave's 32 centroids
                const int64_t row = (int64_t)tm * QT + ra * 32 + l32;
                if (half == 0 && row < nq) {
                    out[row * ldo + (sched.streamed_tile(j) * 8 + wave)] = best;
                }
            }
        } else {
            // Every run that may hold a score <= tau goes to the wavefront's queue in LDS, compacted over the lanes
            // (nearly every run has SOME lane that passes -- 64 lanes, 64 queries -- but only one or two do: stored
            // from their own lanes the records would cost a vector-memory instruction per run for a couple of active
            // lanes); full batches of 64 leave for the rows' record buffers with one atomic and two stores per lane.
            const uint32_t colv = (uint32_t)(col0 + flt.col_base);
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                const float tv = perq[ra * 32 + l32];
                const uint32_t row = (uint32_t)(tm * QT + ra * 32 + l32);
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float u[4];
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        u[t] = __builtin_fmaf(cnv[g][t], -0.5f, acc[ra][4 * g + t]);
                    }
                    const float m = fmaxf(fmaxf(u[0], u[1]), fmaxf(u[2], u[3]));
                    const bool pass = m >= tv && col0 + 8 * g < nb;
                    const unsigned long long mask = __builtin_amdgcn_ballot_w64(pass);
                    if (mask != 0) {
                        if (qcount > kQueueRecords - 64) {
                            flush_queue();
                        }
                        const int at = qcount + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                         __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                        if (pass) {
                            queue[2 * at] = make_uint4(__float_as_uint(acc[ra][4 * g]), __float_as_uint(acc[ra][4 * g + 1]),
                                                       __float_as_uint(acc[ra][4 * g + 2]), __float_as_uint(acc[ra][4 * g + 3]));
                            queue[2 * at + 1] = make_uint4(colv + 8 * g, row, 0u, 0u);
                        }
                        qcount += __builtin_popcountll(mask);
                    }
                }
            }
        }
        if (!has_next) {
            break;
        }
        it_t = n_it;
        tm = n_tm;
        j = n_j;
        jend = n_jend;
        cur = nxt;
    }
    if constexpr (MODE == kRecords) {
        flush_queue();
    }
}

int device_cus()
{
    static std::atomic<int> known{0};
    int cus = known.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        IXA_HIP(hipGetDevice(&dev));
        IXA_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        known.store(cus, std::memory_order_relaxed);
    }
    return cus;
}

// rounds of work items x (loading the query tile + walking a segment), in units of one block-row of matrix work;
// load = what a query tile costs to load, in tiles' time (measured inside the kernel: 1.6 where a tile has the record
// epilogue behind it, about 3 where it has the minima's)
double plan_cost(int64_t tiles_m, int64_t own_n, int64_t wpx, int ra, int64_t seg, double load)
{
    const int64_t S = tiles_m > 0 && wpx / tiles_m > 1 ? wpx / tiles_m : 1;
    const int64_t nseg = (own_n + S * seg - 1) / (S * seg) * S;
    const int64_t rounds = (tiles_m * nseg + wpx - 1) / wpx;
    return (double)rounds * ra * (load + (double)seg);
}

template <int NHS, int PF, int RA, int MODE>
void launch_shape(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, const float *cnp, int64_t nb, const float *qn,
                  const float *test, int metric, float *out, int64_t ldo, ScoreFilter<float> flt, int seg, bool own_resident,
                  hipStream_t s)
{
    constexpr int QT = RA * 32;
    constexpr size_t smem = (size_t)QT * NHS * 32 + QT * 4 + (MODE == kRecords ? kWaves * kQueueRecords * 32 : 0);
    if constexpr (smem > 160 * 1024) {
        fail(kErrInner, "resident coarse kernel: tile of %d queries does not fit LDS", QT);   // the plan never picks it
    } else {
    auto kern = resident_bf16_kernel<NHS, PF, RA, MODE>;
    static std::atomic<bool> configured{false};
    if (!configured) {
        hipFuncAttributes attr;
        IXA_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kern)));
        IXA_REQUIRE(attr.sharedSizeBytes == 0, kErrInner, "resident coarse kernel: unexpected static LDS of %zu bytes",
                    (size_t)attr.sharedSizeBytes);
        IXA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        configured = true;
    }
    const int64_t tiles_m = (nq + QT - 1) / QT, ntiles = (nb + kI8TileRows - 1) / kI8TileRows;
    const unsigned grid = (unsigned)((device_cus() + 7) / 8 * 8);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kWaves * 64), smem, s, Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt,
                       (int)tiles_m, (int)ntiles, seg, own_resident ? 1 : 0);
    }
}

template <int NHS, int PF, int MODE>
void launch_ra(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, const float *cnp, int64_t nb, const float *qn,
               const float *test, int metric, float *out, int64_t ldo, ScoreFilter<float> flt, hipStream_t s)
{
    // tile height, segment length and which operand's tiles an XCD owns, by the number of rounds the launch will take
    const int64_t wpx = (device_cus() + 7) / 8, ntiles = (nb + kI8TileRows - 1) / kI8TileRows;
    const double load = MODE == kRecords ? 1.6 : 3.0;
    int best_ra = 4;
    int64_t best_seg = 1;
    bool best_own = false;
    double best = 1e300;
    for (int ra = 4; ra <= 6; ra++) {
        if ((size_t)ra * 32 * NHS * 32 + ra * 128 + (MODE == kRecords ? kWaves * kQueueRecords * 32 : 0) > 160 * 1024) {
            continue;
        }
        const int64_t tiles_m = (nq + ra * 32 - 1) / (ra * 32);
        for (int own = 0; own < 2; own++) {
            // the XCD with most to do: every resident tile and an eighth of the streamed ones, or the other way round
            const int64_t tm = own ? (tiles_m + 7) / 8 : tiles_m, tn = own ? ntiles : (ntiles + 7) / 8;
            for (int64_t seg = 1;; seg *= 2) {
                const int64_t sg = seg < tn ? seg : tn;   // 1, 2, 4, ... and the XCD's whole share
                const double c = plan_cost(tm, tn, wpx, ra, sg, load);
                if (c < best) {
                    best = c;
                    best_ra = ra;
                    best_seg = sg;
                    best_own = own != 0;
                }
                if (seg >= tn) {
                    break;
                }
            }
        }
    }
    const int seg = (int)best_seg;
    if (best_ra == 4) {
        launch_shape<NHS, PF, 4, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, seg, best_own, s);
    } else if (best_ra == 5) {
        launch_shape<NHS, PF, 5, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, seg, best_own, s);
    } else {
        launch_shape<NHS, PF, 6, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, seg, best_own, s);
    }
}

template <int MODE>
bool launch_for_row(int d3, const uint16_t *Qs, int64_t nq, const uint16_t *Bt, const float *cnp, int64_t nb,
                    const float *qn, const float *test, int metric, float *out, int64_t ldo, ScoreFilter<float> flt,
                    hipStream_t s)
{
    // d3 = 3 dp bf16 per split row, dp = the dimension rounded up to 32: 64, 96 and 128 dimensions
    switch (d3) {
    case 192: launch_ra<12, 4, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, s); return true;
    case 288: launch_ra<18, 6, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, s); return true;
    case 384: launch_ra<24, 8, MODE>(Qs, nq, Bt, cnp, nb, qn, test, metric, out, ldo, flt, s); return true;
    default: return false;
    }
}

}  // namespace

bool resident_coarse_serves(int d3) { return d3 == 192 || d3 == 288 || d3 == 384; }

bool launch_resident_bf16_minima(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, int64_t nb, int d3, const float *qn,
                                 const float *cn_padded, int metric, float *out, int64_t ldo, hipStream_t s)
{
    if (nq <= 0 || nb <= 0 || nb % kI8TileRows != 0 || reinterpret_cast<uintptr_t>(Qs) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(Bt) % 16 != 0 || reinterpret_cast<uintptr_t>(cn_padded) % 16 != 0) {
        return false;
    }
    return launch_for_row<kMinima>(d3, Qs, nq, Bt, cn_padded, nb, qn, nullptr, metric, out, ldo, ScoreFilter<float>{}, s);
}

bool launch_resident_bf16_records(const uint16_t *Qs, int64_t nq, const uint16_t *Bt, int64_t nb, int d3, const float *qn,
                                  const float *cn_padded, int metric, const float *test, ScoreFilter<float> flt,
                                  hipStream_t s)
{
    if (nq <= 0 || nb <= 0 || nb % 4 != 0 || !test || !resident_coarse_serves(d3) ||
        reinterpret_cast<uintptr_t>(Qs) % 16 != 0 || reinterpret_cast<uintptr_t>(Bt) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(cn_padded) % 16 != 0) {
        return false;
    }
    return launch_for_row<kRecords>(d3, Qs, nq, Bt, cn_padded, nb, qn, test, metric, nullptr, 0, flt, s);
}

}  // namespace ixa
