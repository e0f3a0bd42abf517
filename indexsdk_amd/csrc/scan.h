// Host launcher of the fused LUT + ADC scan + top-k kernel.
#pragma once
#include "common.h"

namespace ixa {

// Code layout 2 ("xor48", M = 48, fp32 LUT): byte j of the slot at list position p holds sub-quantizer
//   j < 32:  (j ^ p) & 31              (the 32 lanes of a half wavefront read 32 different ones)
//   j >= 32: 32 + ((j ^ p) & 15)       (16 different ones; lanes 0..15 and 16..31 read two LUT copies)
// The LUT row of a codeword is 64 words: sub-quantizers 0..31, then 32..47 twice.  A lane's word in
// the row is then (c ^ (p & 31)) + block offset with a per-step constant c, whatever the code value:
// conflict-free, and no table of rotation offsets has to live in registers.
__host__ __device__ inline int xor48_sq_of_byte(int j, int p) { return j < 32 ? ((j ^ p) & 31) : 32 + ((j ^ p) & 15); }
__host__ __device__ inline int xor48_byte_of_sq(int m, int p) { return m < 32 ? ((m ^ p) & 31) : 32 + ((m ^ p) & 15); }

struct ScanParams {
    // query side
    const float *queries;      // [nq][d]
    const int32_t *probes;     // [nq][nprobe] list ids, best first; an id outside [0, nlist) (-1 by convention) = none
    int nprobe;
    // trained state
    const float *codebook;     // [M][256][dsub]
    const float *cb_norms;     // [M][256]  |codeword|^2, left-to-right fp32
    int d, M, dsub, metric;
    int lut_fp16;              // 1: LUT entries rounded to IEEE half (RNE), accumulated in fp32
    // inverted lists (arena)
    const uint8_t *codes;
    const int64_t *ids;
    const int64_t *list_off;   // first slot of each list
    const int32_t *list_len;   // valid entries of each list
    int nlist;                 // number of lists
    int code_layout;           // 0 = row, 1 = rot32, 2 = xor48
    // selection
    int k;
    int nsplit;                // workgroups per query; > 1 needs `partial`
    unsigned long long *partial;  // [nq][nsplit][k] keys
    float *out_dist;           // [nq][k]
    int64_t *out_labels;       // [nq][k]
    // scheduling
    const int32_t *order;      // optional permutation of the queries (execution order), may be null
    int xcd_chunks;            // 1: deal contiguous chunks of the execution order to the 8 XCDs
    int64_t nq;                // filled by launch_scan()
    // filled by plan_scan()
    int waves, shared_pool, cap, merge_n, table_n, off_query, off_pools, off_merge, off_table, off_hist, off_misc;
};

// Computes the LDS plan of a launch; returns the dynamic LDS bytes it needs.
size_t plan_scan(ScanParams &p);

void launch_scan(ScanParams p, int64_t nq, hipStream_t s);

// The LDS plan of a launch (host only).  waves = 0: the plan plan_scan() chooses; else the layout for that
// workgroup size (4, 8, 16 wavefronts) and pool kind.  Returns the dynamic LDS bytes; *ctl_bytes = size of the
// shared pool's control block, which follows the 2 x waves words at off_misc.
size_t scan_lds_plan(int d, int M, int lut_fp16, int code_layout, int nprobe, int nsplit, int k, int waves,
                     int shared_pool, ScanParams *out, int *ctl_bytes);

// order[0 .. nq) = the queries grouped by the lists they probe (class = hash of the smallest probed list id).
// cls, hist, cursor as below.
void launch_order_by_locality(const int32_t *probes, int64_t nq, int nprobe, int32_t *cls, int32_t *hist,
                              int32_t *cursor, int32_t *order, hipStream_t s);

// order[0 .. nq) = the queries by descending work class (work = sum of the probed lists' lengths, at most
// max_work).  cls: nq ints; hist: 1024 ints that are ZERO on entry and zero again afterwards;
// cursor: 1024 ints (scratch).
void launch_order_by_work(const int32_t *probes, int64_t nq, int nprobe, const int32_t *list_len, int nlist, long long max_work,
                          int32_t *cls, int32_t *hist, int32_t *cursor, int32_t *order, hipStream_t s);

// *out += sum over probes of list_len[probe]  (a probe outside [0, nlist) contributes nothing).
void launch_count_scanned(const int32_t *probes, int64_t n, const int32_t *list_len, int nlist, unsigned long long *out,
                          hipStream_t s);

}  // namespace ixa
