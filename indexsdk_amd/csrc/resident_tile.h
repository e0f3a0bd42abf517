// Pieces shared by the resident-operand score kernels (flat_i8.hip, coarse_resident.hip): one operand tile lives in
// LDS as [16-byte chunk of K][row][16 B] for the lifetime of a work item, the other operand is read from a tiled
// array (blocks of 32 rows stored as [chunk][row][16 B], flat_i8.h) straight into registers, and the matrix
// instructions of a tile are fully unrolled.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace ixa {

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// N 128-bit LDS reads of consecutive 32-row blocks (512 bytes apart) and the wait for them are inline assembly: the
// compiler's own bookkeeping would wait for a read right after issuing it.  LDS reads complete in order, so "at most N
// outstanding" after the N reads of the next group have been issued means that this group has arrived; the registers
// pass through the wait statement so that no use of them can be scheduled ahead of it.  Other LDS or scalar-memory
// operations in flight can only make such a wait stricter than needed, never weaker.
template <int N, int OFF, int I = 0, typename V>
__device__ __forceinline__ void lds_read_group(uint32_t addr, V (&f)[N])
{
    if constexpr (I < N) {
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f[I]) : "v"(addr), "n"(OFF + 512 * I));
        lds_read_group<N, OFF, I + 1>(addr, f);
    }
}
// (volatile statements keep their order: every register passes through a statement that follows the wait)
template <int N, int PENDING, int I = 0, typename V>
__device__ __forceinline__ void lds_wait_group(V (&f)[N])
{
    if constexpr (I == 0) {
        asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f[0]) : "n"(PENDING));
        lds_wait_group<N, PENDING, 1>(f);
    } else if constexpr (I < N) {
        asm volatile("" : "+v"(f[I]));
        lds_wait_group<N, PENDING, I + 1>(f);
    }
}

// The resident tile: rows first .. first + QT - 1 of a row-major array (rows of D bytes; rows past the end of the array
// repeat its last row) into LDS as [16-byte chunk][row][16 B].  A wavefront moves 16 rows x 4 chunks per step: 64
// contiguous bytes of every row on the memory side, 256 contiguous bytes per chunk on the LDS side (a four-way bank
// conflict; row-fastest would read 16 bytes per row, chunk-fastest would put 64 lanes on four banks), and a
// thread issues eight loads before the first store, so the tile costs a few memory round trips, not one per step.
template <int QT, int D, int NT, int kBatch = 8>
__device__ __forceinline__ void load_resident_tile(unsigned char *lds, const unsigned char *__restrict__ rows, int64_t first,
                                                   int64_t nrows, int tid)
{
    static_assert(QT % 16 == 0 && D % 64 == 0, "tile shape");
    constexpr int kSteps = (QT / 16) * (D / 64);   // wavefront steps of 16 rows x 4 chunks
    constexpr int kWavesT = NT / 64;
    constexpr int kPerWave = (kSteps + kWavesT - 1) / kWavesT;
    const int lane = tid & 63, wave = tid >> 6;
    const int qq = lane & 15, cc = lane >> 4;
    // kBatch = loads in flight per thread (8 where registers are scarce at the call)
#pragma unroll
    for (int i0 = 0; i0 < kPerWave; i0 += kBatch) {
        uint4 v[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            const int step = wave + (i0 + b) * kWavesT;
            const int qb = step % (QT / 16), cb = step / (QT / 16);
            if (i0 + b < kPerWave && step < kSteps) {
                int64_t row = first + qb * 16 + qq;
                row = row < nrows ? row : nrows - 1;
                v[b] = *reinterpret_cast<const uint4 *>(rows + row * D + (cb * 4 + cc) * 16);
            }
        }
#pragma unroll
        for (int b = 0; b < kBatch; b++) {
            const int step = wave + (i0 + b) * kWavesT;
            const int qb = step % (QT / 16), cb = step / (QT / 16);
            if (i0 + b < kPerWave && step < kSteps) {
                *reinterpret_cast<uint4 *>(lds + (cb * 4 + cc) * (QT * 16) + (qb * 16 + qq) * 16) = v[b];
            }
        }
    }
}

// Work items of a persistent launch: XCD x (workgroup b runs on XCD b % 8) owns tiles x, x + 8, ... of the streamed
// operand; an item is (resident tile, segment of the XCD's tiles), resident tile fastest, dealt round-robin to the
// XCD's workgroups.  The S = wpx / tiles_m segments that are in flight together INTERLEAVE tile by tile inside a
// group of S * seg_tiles tiles (segment `sub` of group g takes tiles g * S * seg_tiles + sub, + S, + 2 S, ...): all
// workgroups of the XCD then read the same few tiles at any moment and its L2 holds them for every reader.
// With own_resident the roles are swapped: XCD x owns the RESIDENT tiles x, x + 8, ... and walks every streamed tile
// (fewer, longer items: the choice for launches with few streamed tiles per XCD, where loading the resident tile
// costs more than walking a segment).  streamed_tile(j) / the tm that range() returns are the tiles' real numbers.
struct ResidentItems {
    int tiles_m, own_n, wpx, S, group_tiles, items;
    int tm_add, tm_mul, j_add, j_mul;
    __device__ ResidentItems(int tiles_m_, int ntiles, int seg_tiles, int xcd, int wpx_, bool own_resident = false)
    {
        wpx = wpx_;
        if (own_resident) {
            tiles_m = tiles_m_ > xcd ? (tiles_m_ - xcd + 7) / 8 : 0;
            own_n = ntiles;
            tm_add = xcd, tm_mul = 8, j_add = 0, j_mul = 1;
        } else {
            tiles_m = tiles_m_;
            own_n = ntiles > xcd ? (ntiles - xcd + 7) / 8 : 0;
            tm_add = 0, tm_mul = 1, j_add = xcd, j_mul = 8;
        }
        S = tiles_m > 0 && wpx / tiles_m > 1 ? wpx / tiles_m : 1;
        group_tiles = S * seg_tiles;
        items = tiles_m * ((own_n + group_tiles - 1) / group_tiles * S);
    }
    __device__ int64_t streamed_tile(int j) const { return j_add + (int64_t)j_mul * j; }
    // resident tile, first streamed tile, tile after the last of an item (tiles advance by S); may be empty
    __device__ void range(int it, int &tm, int &j0, int &j1) const
    {
        tm = tm_add + tm_mul * (it % tiles_m);
        const int seg = it / tiles_m, g = seg / S, sub = seg % S;
        j0 = g * group_tiles + sub;
        j1 = (g + 1) * group_tiles < own_n ? (g + 1) * group_tiles : own_n;
    }
    // the first item at or after `it` of the sequence it, it + wpx, ... that has a tile, or -1
    __device__ int next(int it) const
    {
        for (; it < items; it += wpx) {
            int tm, j0, j1;
            range(it, tm, j0, j1);
            if (j0 < j1) {
                return it;
            }
        }
        return -1;
    }
};

}  // namespace ixa
