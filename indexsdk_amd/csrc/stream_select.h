// Streaming brute-force selection: the best `ncand` base rows for every query row, kept as sorted
// keys, without ever materialising more than a bounded stretch of the score matrix.
#pragma once
#include "coarse.h"

namespace ixa {

template <typename S>
struct StreamSelectWorkspace {
    DeviceBuffer<S> scores, tau, thr;
    DeviceBuffer<int32_t> cnt;                    // per-query admitted-candidate counters + overflow flag
    DeviceBuffer<unsigned long long> filter;
    bool cnt_zero = false;                        // every counter is zero (the sampled-bound plan keeps them so)
};

// running[nq][ncand] is written only: once the work queued on the stream has run it holds each query's
// best ncand keys (ordered score << 32 | base row), ascending, kEmptyKey-padded.  The call waits for
// the stream only when it used filtered launches (whose overflow flag decides about a second attempt).
// A first stretch of the base goes through a score scratch of at most scratch_bytes and seeds
// the running keys; afterwards the score kernel admits only what beats each query's current
// ncand-th score and the admitted keys are merged.  If a query ever admits more keys than its
// buffer holds (adversarial base order), the whole selection is redone through the scratch.
// Returns the number of score launches.
// With a mask (device memory, one row of mask_stride bytes per query row, bit b % 8 of byte b / 8 set = base row b
// takes part; AscendIndexFlat::search_with_masks, FR/ascend/AscendIndexFlat.h:78-82) every stretch of the
// score matrix is materialised and the scores of the rows a query leaves out are overwritten with the
// worst score before the selection reads them; keys with that score may come back when fewer than ncand
// rows take part (the caller drops them).
int stream_select_f32(const float *Q, int64_t nq, const float *B, int64_t nb, int d, const float *qn, const float *bn,
                      int metric, int ncand, unsigned long long *running, StreamSelectWorkspace<float> &ws,
                      int64_t scratch_bytes, hipStream_t s, const uint8_t *mask = nullptr, int64_t mask_stride = 0);
// Same selection with approximate scores: Qs / Bs are the bf16 x 3 splits of the operands (rows of d3
// bf16 elements, see launch_split_bf16x3), qn / bn the exact fp32 norms.  Returns -1 without doing
// anything when the shape does not qualify for the bf16 matrix-core kernel.
int stream_select_bf16x3(const uint16_t *Qs, int64_t nq, const uint16_t *Bs, int64_t nb, int d3, const float *qn,
                         const float *bn, int metric, int ncand, unsigned long long *running,
                         StreamSelectWorkspace<float> &ws, int64_t scratch_bytes, hipStream_t s);
// The same selection without a score matrix: the score kernel's admission bound comes from group minima
// over a seed stretch of the base (a bound that holds with overwhelming probability when base rows come in
// no particular order), the admitted scores are appended as records, and every row's result is PROVEN
// afterwards; rows without proof are appended to flag[1 + flag[0]++] (flag: 1 + nq ints, flag[0] zero or the
// count so far) with kEmptyKey in their last key, for the caller's exact plan.  Never waits for the stream.
// Returns -1 without doing anything when the plan does not apply (short bases, small products, more than
// 384 keys, unaligned operands, a scratch too small for 128 rows of records).
// With `refine` the call ends in the exact best-nout SET of every row instead (refine->out_ids[nq][nout],
// unordered; see launch_fold_refine_boundary) and `running` is not touched.
struct BoundaryRefine {
    const float *Q, *C;   // fp32 operands: queries [nq][d], base rows [nb][d]
    int d, nout;
    float cmax, err_scale, round_scale;
    int32_t *out_ids;
};
// With `resident` (and an instance of the resident-query kernel for d3) the two score launches read the base side
// from matrix-core order instead (launch_resident_bf16_minima / _records in coarse.h); same plan, same proofs.
struct ResidentCoarse {
    const uint16_t *Bt;       // base-side split rows, tiled, zero rows up to a whole tile of 256
    const float *cn_padded;   // |c|^2 (zeros for inner product), +inf up to a whole tile
    float cmax;               // largest |c|
};
int stream_select_bf16x3_sampled(const uint16_t *Qs, int64_t nq, const uint16_t *Bs, int64_t nb, int d3,
                                 const float *qn, const float *bn, int metric, int ncand, unsigned long long *running,
                                 StreamSelectWorkspace<float> &ws, int64_t scratch_bytes, int *flag,
                                 const BoundaryRefine *refine, hipStream_t s, const ResidentCoarse *resident = nullptr);
// B: the base in matrix-core order and bn its norms padded with kI8PadNorm to whole tiles of 256 rows (flat_i8.h)
int stream_select_i8(const int8_t *Q, int64_t nq, const int8_t *B, int64_t nb, int d, const int32_t *qn,
                     const int32_t *bn, int ncand, unsigned long long *running, StreamSelectWorkspace<int32_t> &ws,
                     int64_t scratch_bytes, hipStream_t s, const uint8_t *mask = nullptr, int64_t mask_stride = 0);

// scores[r][c] (nq rows of ld, columns [0, nc) standing for base rows col0 + c) = the worst score wherever bit
// col0 + c of the row's mask is clear; the mask row of score row r is row_map[r], or r without a map.
void launch_apply_mask(float *scores, int64_t nq, int64_t ld, int64_t nc, const uint8_t *mask, int64_t mask_stride,
                       const int64_t *row_map, int64_t col0, hipStream_t s);
void launch_apply_mask(int32_t *scores, int64_t nq, int64_t ld, int64_t nc, const uint8_t *mask, int64_t mask_stride,
                       const int64_t *row_map, int64_t col0, hipStream_t s);
// keys[i] = kEmptyKey where its score is the worst score of S (float: +inf, int32: INT32_MAX)
void launch_drop_worst_keys_f32(unsigned long long *keys, int64_t n, hipStream_t s);
void launch_drop_worst_keys_i32(unsigned long long *keys, int64_t n, hipStream_t s);

// idx[i] = row index of keys[i], or -1 for an empty key.
void launch_keys_to_idx(const unsigned long long *keys, int64_t n, int32_t *idx, hipStream_t s);

}  // namespace ixa
