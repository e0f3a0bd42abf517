// int8 Flat: exact int32 L2 scores on the int8 matrix cores, read from the tiled base of flat_i8.h.
//
// resident_i8_kernel -- the query tile stays in LDS, the base goes from memory straight into registers:
//   * a workgroup of 8 wavefronts (two per SIMD) is persistent, one per CU.  It copies a tile of QT = 256 (128
//     for more than 512 dimensions) queries into LDS ONCE, as [16-byte chunk of K][query][16 B], and then walks
//     256-row tiles of the base with it: only base bytes move in the steady state, half of what a kernel that
//     streams both operands needs, and the LDS is never written while it is read: no workgroup barrier and no
//     ring bookkeeping in the main loop;
//   * wavefront w owns base rows 32 w .. 32 w + 31 of the tile and ALL queries: per K-step of 32 bytes it loads
//     ONE operand fragment of the base (1 KB, contiguous in the tiled layout) with one global_load_dwordx4,
//     PF K-steps ahead, into a ring of registers, reads the query fragments from LDS in quads of four 128-bit
//     reads, one quad ahead of the matrix instructions that consume them, and issues RA = QT / 32 of
//     v_mfma_i32_32x32x32_i8; a base byte is fetched by exactly one wavefront of the workgroup;
//   * the base fragment is the first matrix operand, so a lane owns ONE query per accumulator block and 16 base
//     rows.  Filtered launches start the accumulators from floor(-|b|^2 / 2) instead of zero: the block's
//     admission test  |b|^2 - 2 q.b <= thr  becomes  max over the lane's 16 registers >= floor(-thr / 2)
//     (a superset test: exact up to the parity of |b|^2) -- eight v_max3 and one compare per block, with no
//     per-score arithmetic.  The block that passes is re-tested score by score in exact integers from the
//     accumulator and ONE bit per base row (the parity of its norm: distance = |q|^2 - 2 acc - parity), with the
//     query's bound and norm read from LDS: no memory access, so the loads in flight stay in flight;
//   * admitted keys go to a small per-wavefront queue in LDS and leave for the candidate buffers 64 at a time
//     (one atomic per key, issued by 64 lanes together): a wavefront waits for an atomic's round trip once per
//     64 admissions instead of once per admission;
//   * XCD x owns base tiles x, x + 8, ...; its workgroups take (query tile, segment of base tiles) items with
//     the query tile fastest, so the workgroups that run together read the same base tiles and the XCD's L2
//     serves all but the first.
#include "flat_i8.h"
#include "resident_tile.h"
#include "topk.h"

namespace ixa {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }

// ---- layout kernels ------------------------------------------------------------------------------------------------

// one thread per (row, 16-byte chunk)
__global__ __launch_bounds__(256) void i8_tile_rows_kernel(const int8_t *__restrict__ x, int64_t n, int d, int dpad,
                                                           int8_t *__restrict__ tiled, int64_t first)
{
    const int chunks = dpad / 16;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n * chunks) {
        return;
    }
    const int64_t r = e / chunks;
    const int c = (int)(e % chunks);
    const int8_t *src = x + r * d + c * 16;
    uint32_t w[4] = {0, 0, 0, 0};
    if (c * 16 + 16 <= d && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
        const uint4 v = *reinterpret_cast<const uint4 *>(src);
        w[0] = v.x;
        w[1] = v.y;
        w[2] = v.z;
        w[3] = v.w;
    } else {
        for (int t = 0; t < 16; t++) {
            if (c * 16 + t < d) {
                w[t >> 2] |= (uint32_t)(uint8_t)src[t] << (8 * (t & 3));
            }
        }
    }
    *reinterpret_cast<uint4 *>(tiled + i8_tiled_offset(first + r, c, dpad)) = make_uint4(w[0], w[1], w[2], w[3]);
}

__global__ __launch_bounds__(256) void i8_untile_rows_kernel(const int8_t *__restrict__ tiled, int64_t first, int64_t n,
                                                             int d, int dpad, int8_t *__restrict__ out)
{
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < n * d) {
        const int64_t r = e / d;
        const int j = (int)(e % d);
        out[e] = tiled[i8_tiled_offset(first + r, j >> 4, dpad) + (j & 15)];
    }
}

__global__ __launch_bounds__(64) void i8_move_rows_kernel(int8_t *__restrict__ tiled, int dpad, int64_t *__restrict__ ids,
                                                          int32_t *__restrict__ norms, const int64_t *__restrict__ moves)
{
    const int64_t dst = moves[2 * (int64_t)blockIdx.x], src = moves[2 * (int64_t)blockIdx.x + 1];
    for (int c = threadIdx.x; c < dpad / 16; c += 64) {
        *reinterpret_cast<uint4 *>(tiled + i8_tiled_offset(dst, c, dpad)) =
            *reinterpret_cast<const uint4 *>(tiled + i8_tiled_offset(src, c, dpad));
    }
    if (threadIdx.x == 0) {
        ids[dst] = ids[src];
        norms[dst] = norms[src];
    }
}

__global__ __launch_bounds__(256) void i8_pad_norms_kernel(int32_t *__restrict__ norms, int64_t from, int64_t to)
{
    const int64_t i = from + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < to) {
        norms[i] = kI8PadNorm;
    }
}

// ---- plain tile kernel: any dimension, any size ------------------------------------------------------------------------
// 128 x 128 tile per workgroup, 64 x 64 per wavefront as 2 x 2 blocks of v_mfma_i32_32x32x32_i8; K-steps of 64 bytes
// staged in LDS with an 80-byte row stride (conflict-free 128-bit reads).  Serves what the resident kernel does not.
constexpr int kTile = 128;
constexpr int kKBytes = 64;
constexpr int kRowStride = 80;

template <bool VEC16>
__device__ __forceinline__ uint4 load_k16(const int8_t *row, int k, int d)
{
    if (VEC16) {
        if (k < d) {
            return *reinterpret_cast<const uint4 *>(row + k);
        }
        return make_uint4(0, 0, 0, 0);
    }
    uint32_t w[4] = {0, 0, 0, 0};
    for (int t = 0; t < 16; t++) {
        if (k + t < d) {
            w[t >> 2] |= (uint32_t)(uint8_t)row[k + t] << (8 * (t & 3));
        }
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __forceinline__ uint4 load_tiled16(const int8_t *tiled, int64_t row, int k, int dpad)
{
    if (k < dpad) {
        return *reinterpret_cast<const uint4 *>(tiled + i8_tiled_offset(row, k >> 4, dpad));
    }
    return make_uint4(0, 0, 0, 0);
}

template <bool VEC16, bool FILTER>
__global__ __launch_bounds__(256) void score_tile_i8_kernel(const int8_t *__restrict__ Q, int64_t nq,
                                                            const int8_t *__restrict__ Bt, int64_t r0, int64_t r1, int d,
                                                            int dpad, const int32_t *__restrict__ qn,
                                                            const int32_t *__restrict__ bn, int32_t *__restrict__ out,
                                                            int64_t ldo, int tiles_m, int tiles_n,
                                                            ScoreFilter<int32_t> flt)
{
    __shared__ __align__(16) unsigned char As[2][kTile * kRowStride];
    __shared__ __align__(16) unsigned char Bs[2][kTile * kRowStride];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int half = lane >> 5, l32 = lane & 31;
    // 8 consecutive workgroups (one per XCD) take 8 different base tiles; each XCD then walks all
    // query tiles of its base tile, so a base tile is fetched from HBM once and re-used from L2
    const int64_t gs = (int64_t)8 * tiles_m;
    const int64_t grp = blockIdx.x / gs, rem = blockIdx.x % gs;
    const int64_t tile_n = grp * 8 + (rem & 7), tile_m = rem >> 3;
    if (tile_n >= tiles_n) {
        return;
    }
    const int64_t i0 = tile_m * kTile, j0 = r0 + tile_n * kTile;   // j0: row of the whole base

    const int lrow0 = tid >> 2, lrow1 = (tid + 256) >> 2, lk = (tid & 3) * 16;
    const int64_t qa0 = i0 + lrow0 < nq ? i0 + lrow0 : nq - 1, qa1 = i0 + lrow1 < nq ? i0 + lrow1 : nq - 1;
    const int64_t ba0 = j0 + lrow0 < r1 ? j0 + lrow0 : r1 - 1, ba1 = j0 + lrow1 < r1 ? j0 + lrow1 : r1 - 1;
    const int8_t *qrow0 = Q + qa0 * d, *qrow1 = Q + qa1 * d;

    v16i acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++) {
#pragma unroll
        for (int b = 0; b < 2; b++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[a][b][r] = 0;
            }
        }
    }
    const int nk = (d + kKBytes - 1) / kKBytes;
    uint4 ra0 = load_k16<VEC16>(qrow0, lk, d), ra1 = load_k16<VEC16>(qrow1, lk, d);
    uint4 rb0 = load_tiled16(Bt, ba0, lk, dpad), rb1 = load_tiled16(Bt, ba1, lk, dpad);
    *reinterpret_cast<uint4 *>(&As[0][lrow0 * kRowStride + lk]) = ra0;
    *reinterpret_cast<uint4 *>(&As[0][lrow1 * kRowStride + lk]) = ra1;
    *reinterpret_cast<uint4 *>(&Bs[0][lrow0 * kRowStride + lk]) = rb0;
    *reinterpret_cast<uint4 *>(&Bs[0][lrow1 * kRowStride + lk]) = rb1;
    __syncthreads();
    for (int ks = 0; ks < nk; ks++) {
        const int buf = ks & 1;
        if (ks + 1 < nk) {
            const int k = (ks + 1) * kKBytes + lk;
            ra0 = load_k16<VEC16>(qrow0, k, d);
            ra1 = load_k16<VEC16>(qrow1, k, d);
            rb0 = load_tiled16(Bt, ba0, k, dpad);
            rb1 = load_tiled16(Bt, ba1, k, dpad);
        }
        v4i a[2][2], b[2][2];
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                // the k index of an operand byte is a function of (lane half, byte position) that is
                // the same for both operands, and integer sums are order-free, so any such
                // assignment gives the exact dot product
                a[blk][kk] = *reinterpret_cast<const v4i *>(
                    &As[buf][(wr * 64 + blk * 32 + l32) * kRowStride + kk * 32 + half * 16]);
                b[blk][kk] = *reinterpret_cast<const v4i *>(
                    &Bs[buf][(wc * 64 + blk * 32 + l32) * kRowStride + kk * 32 + half * 16]);
            }
        }
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
#pragma unroll
            for (int ra = 0; ra < 2; ra++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    acc[ra][rb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ra][kk], b[rb][kk], acc[ra][rb], 0, 0, 0);
                }
            }
        }
        if (ks + 1 < nk) {
            const int nbuf = buf ^ 1;
            *reinterpret_cast<uint4 *>(&As[nbuf][lrow0 * kRowStride + lk]) = ra0;
            *reinterpret_cast<uint4 *>(&As[nbuf][lrow1 * kRowStride + lk]) = ra1;
            *reinterpret_cast<uint4 *>(&Bs[nbuf][lrow0 * kRowStride + lk]) = rb0;
            *reinterpret_cast<uint4 *>(&Bs[nbuf][lrow1 * kRowStride + lk]) = rb1;
        }
        __syncthreads();
    }
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
        const int64_t col = j0 + wc * 64 + rb * 32 + l32;
        const int32_t bnv = col < r1 ? bn[col] : 0;
#pragma unroll
        for (int ra = 0; ra < 2; ra++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int64_t row = i0 + wr * 64 + ra * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (row < nq && col < r1) {
                    const int32_t part = bnv - 2 * acc[ra][rb][r];
                    if (FILTER) {
                        if (part <= flt.thr[row]) {
                            const int pos = atomicAdd(&flt.cnt[row], 1);
                            if (pos < flt.cap) {
                                flt.cand[row * flt.cap + pos] = make_key(part + qn[row], (uint32_t)col);
                            }
                        }
                    } else {
                        out[row * ldo + (col - r0)] = part + qn[row];
                    }
                }
            }
        }
    }
}

// ---- resident-query kernel -----------------------------------------------------------------------------------------

__device__ __forceinline__ int max16(const v16i &a)
{
    int m0 = max(max(a[0], a[1]), a[2]);
    const int m1 = max(max(a[3], a[4]), a[5]);
    const int m2 = max(max(a[6], a[7]), a[8]);
    int m3 = max(max(a[9], a[10]), a[11]);
    const int m4 = max(max(a[12], a[13]), a[14]);
    m0 = max(max(m0, m1), m2);
    m3 = max(max(m3, m4), a[15]);
    return max(m0, m3);
}

constexpr int kResidentWaves = 8;
constexpr int kNoQuery = 1 << 29;     // test value of a query row past the end: no accumulator reaches it
constexpr int kNoRow = -(kI8PadNorm / 2);   // accumulator start of a base row outside the launch's range, as of a row
                                            // past the end of the base: it reaches no bound
constexpr int kQueueKeys = 128;       // per-wavefront queue of admitted keys (16 bytes each); flushed above 64
constexpr int kResidentMetaBytes = 256 * 16;   // {bound, norm, test value, -} per query of the tile
constexpr int kResidentExtraLds = kResidentMetaBytes + kResidentWaves * kQueueKeys * 16;

// NHS: K-steps of 32 bytes per row (d / 32); PF: K-steps the base loads run ahead (divides NHS); RA: query blocks of
// 32 per tile; FILTER: append admitted keys, otherwise store every score.
template <int NHS, int PF, int RA, bool FILTER>
__global__ __launch_bounds__(kResidentWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void resident_i8_kernel(
    const int8_t *__restrict__ Q, int64_t nq, const int8_t *__restrict__ Bt, const int32_t *__restrict__ bn, int64_t r0,
    int64_t r1, const int32_t *__restrict__ qn, int32_t *__restrict__ out, int64_t ldo, ScoreFilter<int32_t> flt,
    int tiles_m, int64_t tile0, int ntiles, int seg_tiles)
{
    constexpr int D = NHS * 32, QT = RA * 32;
    constexpr int QPH = RA / 4;          // quads per K-step
    constexpr int kStepLds = QT * 32;    // LDS bytes of one K-step: two chunks of QT x 16 bytes
    static_assert(NHS % PF == 0 && RA % 4 == 0, "shape");
    extern __shared__ __align__(16) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, l32 = lane & 31;

    const int xcd = blockIdx.x & 7, wi = blockIdx.x >> 3, wpx = gridDim.x >> 3;
    const ResidentItems sched(tiles_m, ntiles, seg_tiles, xcd, wpx);
    const int S = sched.S;
    const int first_item = sched.next(wi);
    if (first_item < 0) {
        return;
    }
    const uint32_t lds_base = (uint32_t)reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)lds);
    const uint32_t a_lane = lds_base + (uint32_t)(half * (QT * 16) + l32 * 16);   // + step * kStepLds + block * 512
    const uint32_t a_lane_hi = a_lane + 65536;
    const unsigned char *Bb = reinterpret_cast<const unsigned char *>(Bt);

    // tile j of this XCD's share -> first row of this wave's 32-row block, and the lane's 16 bytes of its first fragment
    auto block_row0 = [&](int j) { return (tile0 + xcd + 8 * (int64_t)j) * kI8TileRows + wave * 32; };
    auto block_ptr = [&](int j) { return Bb + block_row0(j) * (int64_t)D + lane * 16; };

    v16i acc[RA];
    v4i breg[PF];
    v4i bnv[4];
    int cur_tm = -1;
    // filtered launches: {thr, |q|^2, floor(-thr / 2), -} of the tile's queries behind the query tile (in LDS rather
    // than in registers: the main loop has none to spare), then the wavefronts' key queues
    int4 *meta = reinterpret_cast<int4 *>(lds + QT * D);
    uint4 *queue = reinterpret_cast<uint4 *>(lds + QT * D + kResidentMetaBytes) + wave * kQueueKeys;
    int qcount = 0;   // keys in this wavefront's queue (wave-uniform)
    // every queued key takes its place in its query's candidate buffer; 64 lanes, one key each
    auto flush_queue = [&]() {
        wave_lds_fence();
        for (int i0 = 0; i0 < qcount; i0 += 64) {
            if (i0 + lane < qcount) {
                const uint4 e = queue[i0 + lane];   // {base row, ordered score, query row, -}
                const int pos = atomicAdd(&flt.cnt[e.z], 1);
                if (pos < flt.cap) {
                    flt.cand[(int64_t)e.z * flt.cap + pos] = ((key_t)e.y << 32) | e.x;
                }
            }
        }
        wave_lds_fence();
        qcount = 0;
    };

    int it_t = first_item;
    int tm, j, jend;
    sched.range(it_t, tm, j, jend);
    const unsigned char *cur = block_ptr(j);
    // Loads are issued in the same order here and in the loop -- norms of a tile before its fragments -- so that the
    // wait for the norms at a tile's start leaves the PF fragment loads behind them in flight.
    if constexpr (FILTER) {
        const int32_t *bp = bn + block_row0(j) + 4 * half;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            bnv[g] = *reinterpret_cast<const v4i *>(bp + 8 * g);
        }
        asm volatile("" ::: "memory");
    }
#pragma unroll
    for (int p = 0; p < PF; p++) {
        breg[p] = *reinterpret_cast<const v4i *>(cur + p * 1024);
    }
    bool staggered = false;
    while (true) {
        if (tm != cur_tm) {
            // the query tile: LDS [chunk][query][16 B]; rows past the end of the batch repeat its last row
            if (cur_tm >= 0) {
                __syncthreads();
            }
            load_resident_tile<QT, D, kResidentWaves * 64>(lds, reinterpret_cast<const unsigned char *>(Q),
                                                           (int64_t)tm * QT, nq, tid);
            if constexpr (FILTER) {
                if (tid < QT) {
                    const int64_t row = (int64_t)tm * QT + tid;
                    // a row past the end of the batch gets bounds nothing meets
                    const int32_t thr = row < nq ? flt.thr[row] : 0;
                    meta[tid] = row < nq ? make_int4(thr, qn[row], (-thr) >> 1, 0) : make_int4(-(1 << 30), 0, kNoQuery, 0);
                }
            }
            cur_tm = tm;
            __syncthreads();
            // The two wavefronts of a SIMD (w and w + 4) would otherwise reach the end of every tile together and
            // leave the matrix cores idle while both test their accumulators: the second one starts half a tile
            // late, once, and from then on each one's epilogue runs under the other's matrix instructions.
            if (!staggered && wave >= kResidentWaves / 2) {
                // a wavefront's tile is NHS * RA matrix instructions of 32 cycles, and two wavefronts share the
                // matrix core: half a tile of wall time is 32 NHS RA cycles, s_sleep counts in units of 64
                constexpr int kHalfTile = NHS * RA / 2;
                __builtin_amdgcn_s_sleep(kHalfTile < 127 ? kHalfTile : 127);
            }
            staggered = true;
        }
        // the tile after this one (the last tile names itself: its loads are harmless repeats)
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
        const int32_t *nbp = bn + block_row0(n_j) + 4 * half;

        v16i c0;
        uint32_t par = 0;   // bit 16 + r: parity of the norm of the lane's r-th base row
        if constexpr (FILTER) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                c0[r] = (-bnv[r >> 2][r & 3]) >> 1;   // floor(-|b|^2 / 2)
                par = __builtin_amdgcn_alignbit((uint32_t)bnv[r >> 2][r & 3], par, 1);
            }
            // the first and the last tile of a launch may reach outside [r0, r1): those rows take no part
            const int64_t first_row = block_row0(j);
            if (first_row < r0 || first_row + 32 > r1) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int64_t col = first_row + 4 * half + 8 * (r >> 2) + (r & 3);
                    c0[r] = (col >= r0 && col < r1) ? c0[r] : kNoRow;
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                c0[r] = 0;
            }
        }
        v4i fa[2][4];
        lds_read_group<4, 0>(a_lane, fa[0]);
        static_for<0, QPH * NHS>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            constexpr int hs = u / QPH, p = u % QPH;
            if constexpr (u + 1 < QPH * NHS) {
                constexpr int off = ((u + 1) / QPH) * kStepLds + ((u + 1) % QPH) * 2048;
                if constexpr (off >= 65536) {
                    lds_read_group<4, off - 65536>(a_lane_hi, fa[(u + 1) & 1]);
                } else {
                    lds_read_group<4, off>(a_lane, fa[(u + 1) & 1]);
                }
                lds_wait_group<4, 4>(fa[u & 1]);
            } else {
                lds_wait_group<4, 0>(fa[u & 1]);
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int ra = p * 4 + t;
                acc[ra] = __builtin_amdgcn_mfma_i32_32x32x32_i8(breg[hs % PF], fa[u & 1][t], hs == 0 ? c0 : acc[ra], 0, 0, 0);
            }
            if constexpr (p == QPH - 1) {
                if constexpr (FILTER && hs == NHS - PF) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        bnv[g] = *reinterpret_cast<const v4i *>(nbp + 8 * g);
                    }
                    asm volatile("" ::: "memory");
                }
                if constexpr (hs + PF < NHS) {
                    breg[hs % PF] = *reinterpret_cast<const v4i *>(cur + (hs + PF) * 1024);
                } else {
                    breg[hs % PF] = *reinterpret_cast<const v4i *>(nxt + (hs + PF - NHS) * 1024);
                }
                asm volatile("" ::: "memory");
            }
        });
        // a lane owns query (block ra, l32) and base rows row0 + 8 g + 4 half + t of the wave's block
        const int64_t col0 = block_row0(j) + 4 * half;
        if constexpr (FILTER) {
            // per block: {thr, |q|^2, test value} of the lane's query and ONE compare of the block's largest
            // accumulator with the test value; the lane masks stay in scalar registers
            int4 mt[RA];
            unsigned long long hit[RA], any = 0;
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                mt[ra] = meta[ra * 32 + l32];
            }
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                hit[ra] = __builtin_amdgcn_ballot_w64(max16(acc[ra]) >= mt[ra].z);
                any |= hit[ra];
            }
            if (any != 0) {
                const uint32_t colv = (uint32_t)col0;
#pragma unroll
                for (int ra = 0; ra < RA; ra++) {
                    if (hit[ra] != 0) {
                        const int nthr = -mt[ra].x;   // thr <= 2^28 by the caller's clamp, > INT32_MIN
                        const uint32_t row = (uint32_t)(tm * QT + ra * 32 + l32);
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            // the test value again, register by register (a superset test), then in exact integers:
                            // |b|^2 - 2 q.b = -(2 acc + parity) <= thr  <=>  2 acc + parity >= -thr
                            if (__builtin_amdgcn_ballot_w64(acc[ra][r] >= mt[ra].z) != 0) {
                                const int t2 = (acc[ra][r] << 1) + (int)((par >> (16 + r)) & 1u);
                                const bool pass = t2 >= nthr;
                                const unsigned long long mask = __builtin_amdgcn_ballot_w64(pass);
                                if (mask != 0) {
                                    const int pre = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                                                              __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
                                    if (pass) {
                                        const uint32_t score = (uint32_t)(mt[ra].y - t2) ^ 0x80000000u;   // ordered int32
                                        queue[qcount + pre] = make_uint4(colv + 8 * (r >> 2) + (r & 3), score, row, 0u);
                                    }
                                    qcount += __builtin_popcountll(mask);
                                    if (qcount > kQueueKeys - 64) {
                                        flush_queue();
                                    }
                                }
                            }
                        }
                    }
                }
            }
        } else {
            int32_t bnr[16];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                bnr[r] = bn[col0 + 8 * (r >> 2) + (r & 3)];
            }
#pragma unroll
            for (int ra = 0; ra < RA; ra++) {
                const int64_t row = (int64_t)tm * QT + ra * 32 + l32;
                if (row < nq) {
                    const int32_t qn_row = qn[row];
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int64_t col = col0 + 8 * (r >> 2) + (r & 3);
                        if (col >= r0 && col < r1) {
                            out[row * ldo + (col - r0)] = qn_row + bnr[r] - 2 * acc[ra][r];
                        }
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
    if constexpr (FILTER) {
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

template <int NHS, int PF, int RA, bool FILTER>
void launch_resident(const int8_t *Q, int64_t nq, const int8_t *tiled, const int32_t *qn, const int32_t *bn, int64_t r0,
                     int64_t r1, int32_t *out, int64_t ldo, ScoreFilter<int32_t> flt, hipStream_t s)
{
    constexpr int QT = RA * 32;
    constexpr size_t smem = (size_t)QT * NHS * 32 + (FILTER ? kResidentExtraLds : 0);
    static_assert(smem <= 160 * 1024, "the query tile must fit the LDS of a CU");
    auto kern = resident_i8_kernel<NHS, PF, RA, FILTER>;
    static std::atomic<bool> configured{false};   // per instantiation
    if (!configured) {
        hipFuncAttributes attr;
        IXA_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kern)));
        // the fragment reads address the query tile from LDS offset 0 of the dynamic allocation only
        IXA_REQUIRE(attr.sharedSizeBytes == 0, kErrInner, "resident int8 kernel: unexpected static LDS of %zu bytes",
                    (size_t)attr.sharedSizeBytes);
        IXA_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem));
        configured = true;
    }
    const int64_t tiles_m = (nq + QT - 1) / QT;
    const int64_t tile0 = r0 / kI8TileRows;
    const int64_t ntiles = (r1 + kI8TileRows - 1) / kI8TileRows - tile0;
    IXA_REQUIRE(tiles_m < (1 << 20) && ntiles < ((int64_t)1 << 30), kErrInvalidParam, "int8 score launch too large");
    const unsigned grid = (unsigned)((device_cus() + 7) / 8 * 8);   // one persistent workgroup per CU
    const int64_t wpx = grid / 8, own_n = (ntiles + 7) / 8;
    // segments: enough items for an even share per workgroup, long enough to pay for a query tile that changes
    const int seg = (int)std::min<int64_t>(16, std::max<int64_t>(1, (own_n * tiles_m + wpx * 8 - 1) / (wpx * 8)));
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kResidentWaves * 64), smem, s, Q, nq, tiled, bn, r0, r1, qn, out, ldo, flt,
                       (int)tiles_m, tile0, (int)ntiles, seg);
}

template <bool FILTER>
bool launch_resident_for_dim(int d, const int8_t *Q, int64_t nq, const int8_t *tiled, const int32_t *qn, const int32_t *bn,
                             int64_t r0, int64_t r1, int32_t *out, int64_t ldo, ScoreFilter<int32_t> flt, hipStream_t s)
{
    // the dimensions the reference's Int8Flat serves (FR/ascend/impl/AscendIndexInt8FlatImpl.cpp:55)
    switch (d) {
    case 64: launch_resident<2, 2, 8, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 128: launch_resident<4, 4, 8, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 256: launch_resident<8, 4, 8, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 384: launch_resident<12, 4, 8, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 512: launch_resident<16, 4, 8, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 768: launch_resident<24, 8, 4, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    case 1024: launch_resident<32, 8, 4, FILTER>(Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s); return true;
    default: return false;
    }
}

template <bool FILTER>
void launch_scores(const int8_t *Q, int64_t nq, const int8_t *tiled, int d, const int32_t *qn, const int32_t *bn,
                   int64_t r0, int64_t r1, int32_t *out, int64_t ldo, ScoreFilter<int32_t> flt, hipStream_t s)
{
    if (nq <= 0 || r1 <= r0) {
        return;
    }
    IXA_REQUIRE(r0 >= 0 && reinterpret_cast<uintptr_t>(tiled) % 16 == 0, kErrInner, "int8 base is not tiled storage");
    const bool aligned = reinterpret_cast<uintptr_t>(Q) % 16 == 0 && reinterpret_cast<uintptr_t>(bn) % 16 == 0;
    // launches of a few tiles are served faster by the plain kernel's many small workgroups
    if (aligned && (r1 - r0) >= 8 * kI8TileRows &&
        launch_resident_for_dim<FILTER>(d, Q, nq, tiled, qn, bn, r0, r1, out, ldo, flt, s)) {
        return;
    }
    const int dpad = i8_padded_dim(d);
    const int64_t tiles_m = (nq + kTile - 1) / kTile, tiles_n = (r1 - r0 + kTile - 1) / kTile;
    const int64_t nblocks = (tiles_n + 7) / 8 * 8 * tiles_m;
    IXA_REQUIRE(nblocks < (int64_t)1 << 31, kErrInvalidParam, "score tile grid too large");
    const bool vec = d % 16 == 0 && reinterpret_cast<uintptr_t>(Q) % 16 == 0;
    dim3 grid((unsigned)nblocks), block(256);
    if (vec) {
        hipLaunchKernelGGL((score_tile_i8_kernel<true, FILTER>), grid, block, 0, s, Q, nq, tiled, r0, r1, d, dpad, qn, bn, out,
                           ldo, (int)tiles_m, (int)tiles_n, flt);
    } else {
        hipLaunchKernelGGL((score_tile_i8_kernel<false, FILTER>), grid, block, 0, s, Q, nq, tiled, r0, r1, d, dpad, qn, bn,
                           out, ldo, (int)tiles_m, (int)tiles_n, flt);
    }
}

}  // namespace

bool i8_resident_kernel_serves(int d)
{
    return d == 64 || d == 128 || d == 256 || d == 384 || d == 512 || d == 768 || d == 1024;
}

void launch_i8_tile_rows(const int8_t *x, int64_t n, int d, int8_t *tiled, int64_t first, hipStream_t s)
{
    if (n > 0) {
        const int dpad = i8_padded_dim(d);
        hipLaunchKernelGGL(i8_tile_rows_kernel, dim3(blocks_for(n * (dpad / 16))), dim3(256), 0, s, x, n, d, dpad, tiled,
                           first);
    }
}

void launch_i8_untile_rows(const int8_t *tiled, int64_t first, int64_t n, int d, int8_t *out, hipStream_t s)
{
    if (n > 0) {
        hipLaunchKernelGGL(i8_untile_rows_kernel, dim3(blocks_for(n * d)), dim3(256), 0, s, tiled, first, n, d,
                           i8_padded_dim(d), out);
    }
}

void launch_i8_move_rows(int8_t *tiled, int d, int64_t *ids, int32_t *norms, const int64_t *moves, int64_t nmoves,
                         hipStream_t s)
{
    if (nmoves > 0) {
        hipLaunchKernelGGL(i8_move_rows_kernel, dim3((unsigned)nmoves), dim3(64), 0, s, tiled, i8_padded_dim(d), ids, norms,
                           moves);
    }
}

void launch_i8_pad_norms(int32_t *norms, int64_t from, int64_t to, hipStream_t s)
{
    if (to > from) {
        hipLaunchKernelGGL(i8_pad_norms_kernel, dim3(blocks_for(to - from)), dim3(256), 0, s, norms, from, to);
    }
}

void launch_i8_scores_stored(const int8_t *Q, int64_t nq, const int8_t *tiled, int d, const int32_t *qn,
                             const int32_t *bn, int64_t r0, int64_t r1, int32_t *out, int64_t ldo, hipStream_t s)
{
    launch_scores<false>(Q, nq, tiled, d, qn, bn, r0, r1, out, ldo, ScoreFilter<int32_t>{}, s);
}

void launch_i8_scores_filtered(const int8_t *Q, int64_t nq, const int8_t *tiled, int d, const int32_t *qn,
                               const int32_t *bn, int64_t r0, int64_t r1, ScoreFilter<int32_t> flt, hipStream_t s)
{
    launch_scores<true>(Q, nq, tiled, d, qn, bn, r0, r1, nullptr, 0, flt, s);
}

}  // namespace ixa
