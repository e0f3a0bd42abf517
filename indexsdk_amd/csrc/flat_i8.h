// int8 Flat base in matrix-core order, and the score kernels that read it.
//
// The reference keeps its int8 base in a layout shaped for its matrix unit -- [block of 16 rows][piece of
// 32 bytes of K][16 rows][32 bytes], FR/ascenddaemon/impl/IndexInt8Flat.cpp:173-175, 271-274, and moves
// single vectors inside it piece by piece, :1003-1015; the counterpart here is cut for
// v_mfma_i32_32x32x32_i8: a BLOCK of 32 consecutive rows is stored as [chunk c][row r][16 bytes], chunk c
// holding bytes 16 c .. 16 c + 15 of every row (rows zero-padded to dpad = a multiple of 32 bytes), so
// the operand fragment of a wavefront -- 32 rows x the two chunks of a K-step of 32 -- is 1 KB of
// contiguous memory: lane (row, half) loads its 16 bytes at block + step * 1024 + lane * 16, fully
// coalesced, straight into the registers the matrix instruction reads.
#pragma once
#include "coarse.h"

namespace ixa {

constexpr int kI8BlockRows = 32;
constexpr int kI8TileRows = 256;   // rows a workgroup of the resident kernel takes at a time; buffers are padded to it
// Norm of the padding rows behind the last vector of a tile, and the largest bound a filtered launch may be given: every
// real distance (at most 4096 * 254^2 < 2^28) lies at or below the bound, the "distance" of a padding row (2^30 and
// more) above it, and nothing the kernels compute from either leaves the int32 range.
constexpr int32_t kI8PadNorm = 1 << 30;
constexpr int32_t kI8MaxBound = 1 << 28;

inline int i8_padded_dim(int d) { return (d + 31) / 32 * 32; }
// byte offset of chunk c of a row
__host__ __device__ inline int64_t i8_tiled_offset(int64_t row, int chunk, int dpad)
{
    return (row >> 5) * (32 * (int64_t)dpad) + (int64_t)chunk * 512 + (row & 31) * 16;
}
// bytes of a tiled base of n rows (whole tiles of kI8TileRows rows)
inline size_t i8_tiled_bytes(int64_t n, int d)
{
    return (size_t)round_up(n, kI8TileRows) * (size_t)i8_padded_dim(d);
}

// rows [first, first + n) of the tiled base <- n row-major rows of d bytes (device memory)
void launch_i8_tile_rows(const int8_t *x, int64_t n, int d, int8_t *tiled, int64_t first, hipStream_t s);
// n row-major rows of d bytes <- rows [first, first + n) of the tiled base
void launch_i8_untile_rows(const int8_t *tiled, int64_t first, int64_t n, int d, int8_t *out, hipStream_t s);
// move j: row moves[2 j + 1] (vector, id, norm) over row moves[2 j]; sources and destinations are disjoint
void launch_i8_move_rows(int8_t *tiled, int d, int64_t *ids, int32_t *norms, const int64_t *moves, int64_t nmoves,
                         hipStream_t s);
// norms[i] = kI8PadNorm for i in [from, to): rows past the end of the base inside its last tile never pass a bound
void launch_i8_pad_norms(int32_t *norms, int64_t from, int64_t to, hipStream_t s);

// Exact int32 L2 scores |q|^2 + |b|^2 - 2 q.b of nq row-major queries against rows [r0, r1) of a tiled base
// (FR/ops/ascendc/op_kernel/ascendc_dist_int8_flat_l2.cpp:201-203, 485-500, without its scale-and-round step).
// bn: norms of the whole base, indexed by row and padded with kI8PadNorm up to a multiple of kI8TileRows.
//   stored:   out[row * ldo + (col - r0)]
//   filtered: rows with |b|^2 - 2 q.b <= flt.thr[row] are appended to flt.cand[row][flt.cnt[row]++] as keys
//             (score, col) -- col is the row of the WHOLE base, flt.col_base is not used; flt.thr[row] must not
//             exceed kI8MaxBound - |q|^2
void launch_i8_scores_stored(const int8_t *Q, int64_t nq, const int8_t *tiled, int d, const int32_t *qn,
                             const int32_t *bn, int64_t r0, int64_t r1, int32_t *out, int64_t ldo, hipStream_t s);
void launch_i8_scores_filtered(const int8_t *Q, int64_t nq, const int8_t *tiled, int d, const int32_t *qn,
                               const int32_t *bn, int64_t r0, int64_t r1, ScoreFilter<int32_t> flt, hipStream_t s);
// whether the resident-query kernel serves this dimension (otherwise a plain tile kernel does)
bool i8_resident_kernel_serves(int d);

}  // namespace ixa
