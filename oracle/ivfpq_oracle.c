/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference IVFPQ / Flat search arithmetic.
 *
 * This file is the parity checker for the HIP path and the "port" CPU baseline of the benchmark.
 * Nothing in the shipped library links, loads or calls it; only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may use it.
 *
 * Every function cites the reference code it restates (paths relative to the reference root,
 * FR/ = feature_retrieval/src/ascendfaiss/).  All arithmetic is IEEE fp32 with no FMA contraction
 * (build with -ffp-contract=off) and strictly left-to-right accumulation so that "bit-exact" is
 * well defined across compilers.
 *
 * Pinning status (what independent check fixes each function; see tests/test_oracle_*.py):
 *   orc_sqnorms, orc_coarse_dist ...... closed form vs float64 numpy (||q||^2+||c||^2-2q.c == |q-c|^2)
 *   orc_coarse_probe / orc_assign ..... full stable argsort of the same matrix; brute force
 *   orc_pq_encode ..................... brute-force float64 argmin with tie/near-tie accounting,
 *                                       hand-computed tiny case, first-minimum-wins case
 *   orc_lut ........................... closed form vs float64; q_m == codeword -> ~0
 *   orc_f32_to_f16 / f16_to_f32 ....... numpy.float16 round trip on all 65536 half patterns
 *   orc_search (ADC + top-k) .......... sum_m lut == |q - decode(code)|^2 in float64 (by_residual=false
 *                                       invariant), full-sort ground truth, self-query top-1,
 *                                       FLT_MAX/-1 sentinels, the AICPU top-k test recipe
 *                                       (FR/test/aicpu/test_topk_flat.cc:52-187)
 *   orc_flat_i8 ....................... exact integer closed form vs int64 numpy
 *   orc_flat_f32 ...................... closed form vs float64 numpy + full sort
 *   orc_merge_results ................. stable sort of the device-major concatenation (what a k-way
 *                                       merge with a strict comparison must equal), hand-made case
 *                                       with invalid labels in the middle of a list
 *   orc_kmeans ........................ PARITY UNPINNED against faiss::Clustering (faiss is absent);
 *                                       only Lloyd invariants (objective non-increasing) are checked.
 *                                       Search parity is judged on shared, injected codebooks.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_METRIC_IP 0 /* faiss::METRIC_INNER_PRODUCT */
#define ORC_METRIC_L2 1 /* faiss::METRIC_L2 */

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------ */
/* fp16 helpers (round-to-nearest-even), used only for the fp16-LUT mode.                        */

ORC_API uint16_t orc_f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mant = x & 0x007fffffu;
    int32_t exp = (int32_t)((x >> 23) & 0xff);
    if (exp == 0xff) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (mant ? (0x0200u | (mant >> 13)) : 0));
    }
    int32_t e = exp - 127 + 15;
    if (e >= 0x1f) {
        return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
    }
    if (e <= 0) { /* subnormal half or zero */
        if (e < -10) {
            return (uint16_t)sign;
        }
        mant |= 0x00800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half & 1u))) {
            half++;
        }
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) {
        half++; /* may carry into the exponent, which is the correct behaviour */
    }
    return (uint16_t)(sign | half);
}

ORC_API float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    uint32_t x;
    if (exp == 0) {
        if (mant == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                e++;
                mant <<= 1;
            } while (!(mant & 0x400u));
            mant &= 0x3ffu;
            x = sign | ((uint32_t)(127 - 15 - e) << 23) | (mant << 13);
        }
    } else if (exp == 0x1f) {
        x = sign | 0x7f800000u | (mant << 13);
    } else {
        x = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ------------------------------------------------------------------------------------------ */
/* Norms: FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1114-1126 (sum of val*val, left to right).     */

static float sqnorm(const float *v, int d)
{
    float s = 0.0f;
    for (int j = 0; j < d; j++) {
        float val = v[j];
        s += val * val;
    }
    return s;
}

static float dotp(const float *a, const float *b, int d)
{
    float s = 0.0f;
    for (int j = 0; j < d; j++) {
        s += a[j] * b[j];
    }
    return s;
}

ORC_API void orc_sqnorms(const float *x, int64_t n, int d, float *out)
{
    for (int64_t i = 0; i < n; i++) {
        out[i] = sqnorm(x + i * d, d);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Coarse distance: FR/ops/ascendc/op_kernel/distance_flat_l2_mins_at_fp32.cpp:191-210
 *   dist = broadcast(||q||^2) + ||c||^2, then minus (q.c) twice.  (x - g) - g == x - 2g exactly in
 *   binary floating point unless 2g overflows, so this is written as (qn + cn) - 2*dot.
 * IP (beyond the reference's functional envelope): dist = dot, larger is better.               */

static float coarse_one(const float *q, float qn, const float *c, float cn, int d, int metric)
{
    float g = dotp(q, c, d);
    if (metric == ORC_METRIC_IP) {
        return g;
    }
    float base = qn + cn;
    base = base - g;
    base = base - g;
    return base;
}

ORC_API void orc_coarse_dist(const float *q, int64_t nq, const float *cent, int64_t nlist, int d, int metric,
                             float *out)
{
    float *cn = (float *)malloc(sizeof(float) * (size_t)nlist);
    orc_sqnorms(cent, nlist, d, cn);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nq; i++) {
        float qn = sqnorm(q + i * d, d);
        for (int64_t j = 0; j < nlist; j++) {
            out[i * nlist + j] = coarse_one(q + i * d, qn, cent + j * d, cn[j], d, metric);
        }
    }
    free(cn);
}

/* "a is better than b" for a (distance, sequence) pair; sequence breaks exact ties.             */
static inline int better(float da, int64_t sa, float db, int64_t sb, int metric)
{
    if (da != db) {
        return metric == ORC_METRIC_IP ? (da > db) : (da < db);
    }
    return sa < sb;
}

/* Bounded top-k as a binary heap whose root is the WORST kept element, in the manner of the
 * AICPU heaps (FR/ops/cpukernel/impl/utils/kernel_utils.h:132-157 UpdateHeap) but with a total
 * order (dist, seq) so the result is deterministic.                                            */
typedef struct {
    float d;
    int64_t seq;
    int64_t label;
} orc_ent;

static void heap_sift_down(orc_ent *h, int64_t n, int64_t i, int metric)
{
    for (;;) {
        int64_t l = 2 * i + 1, r = l + 1, w = i;
        if (l < n && better(h[w].d, h[w].seq, h[l].d, h[l].seq, metric)) {
            w = l;
        }
        if (r < n && better(h[w].d, h[w].seq, h[r].d, h[r].seq, metric)) {
            w = r;
        }
        if (w == i) {
            return;
        }
        orc_ent t = h[i];
        h[i] = h[w];
        h[w] = t;
        i = w;
    }
}

static void heap_sift_up(orc_ent *h, int64_t i, int metric)
{
    while (i > 0) {
        int64_t p = (i - 1) / 2;
        if (better(h[p].d, h[p].seq, h[i].d, h[i].seq, metric)) {
            orc_ent t = h[i];
            h[i] = h[p];
            h[p] = t;
            i = p;
        } else {
            return;
        }
    }
}

static inline void heap_offer(orc_ent *h, int64_t *n, int64_t k, float d, int64_t seq, int64_t label, int metric)
{
    if (*n < k) {
        h[*n].d = d;
        h[*n].seq = seq;
        h[*n].label = label;
        heap_sift_up(h, *n, metric);
        (*n)++;
    } else if (better(d, seq, h[0].d, h[0].seq, metric)) {
        h[0].d = d;
        h[0].seq = seq;
        h[0].label = label;
        heap_sift_down(h, k, 0, metric);
    }
}

/* pops into best-first order (final heap sort: topk_flat_fp32_cpu_kernel.cpp:213-220)          */
static void heap_drain_sorted(orc_ent *h, int64_t n, int metric)
{
    for (int64_t end = n - 1; end > 0; end--) {
        orc_ent t = h[0];
        h[0] = h[end];
        h[end] = t;
        heap_sift_down(h, end, 0, metric);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Probe selection: FR/ops/cpukernel/impl/topk_flat_fp32_cpu_kernel.cpp:223-384 with attrs
 * asc=1, k=nprobe (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2127-2136): the nprobe best centroids,
 * best first.  Exact ties resolve to the smaller centroid id.  The reference's 0x7bff heap seed
 * (topk_flat_fp32_cpu_kernel.cpp:253) is a defect and is not reproduced.                        */

ORC_API void orc_coarse_probe(const float *q, int64_t nq, const float *cent, int64_t nlist, int d, int metric,
                              int64_t nprobe, int64_t *out_ids, float *out_dist)
{
    float *cn = (float *)malloc(sizeof(float) * (size_t)nlist);
    orc_sqnorms(cent, nlist, d, cn);
    if (nprobe > nlist) {
        nprobe = nlist;
    }
#pragma omp parallel
    {
        orc_ent *h = (orc_ent *)malloc(sizeof(orc_ent) * (size_t)nprobe);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < nq; i++) {
            const float *qi = q + i * d;
            float qn = sqnorm(qi, d);
            int64_t hn = 0;
            for (int64_t j = 0; j < nlist; j++) {
                float dj = coarse_one(qi, qn, cent + j * d, cn[j], d, metric);
                heap_offer(h, &hn, nprobe, dj, j, j, metric);
            }
            heap_drain_sorted(h, hn, metric);
            for (int64_t r = 0; r < nprobe; r++) {
                out_ids[i * nprobe + r] = h[r].label;
                if (out_dist) {
                    out_dist[i * nprobe + r] = h[r].d;
                }
            }
        }
        free(h);
    }
    free(cn);
}

/* Coarse assignment at add time = nearest centroid under L2
 * (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:603-672; IndexFlatL2::assign or the k=1 device path). */
ORC_API void orc_assign(const float *x, int64_t n, const float *cent, int64_t nlist, int d, int64_t *out)
{
    orc_coarse_probe(x, n, cent, nlist, d, ORC_METRIC_L2, 1, out, NULL);
}

/* ------------------------------------------------------------------------------------------ */
/* PQ encode: FR/ascend/impl/AscendIndexIVFPQImpl.cpp:879-921 (encodeSingleVectorPQ,
 * findCentroidInSubQuantizer, calDistance): raw vector (by_residual = false), direct
 * sum (a-b)^2 left to right, strict '<' so the first minimum wins.                             */

ORC_API void orc_pq_encode(const float *x, int64_t n, int d, int M, const float *codebook, uint8_t *codes)
{
    int dsub = d / M;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        for (int m = 0; m < M; m++) {
            const float *sub = x + i * d + (int64_t)m * dsub;
            const float *cb = codebook + (int64_t)m * 256 * dsub;
            float min_dist = FLT_MAX;
            uint8_t arg = 0;
            for (int k = 0; k < 256; k++) {
                const float *c = cb + (int64_t)k * dsub;
                float dist = 0.0f;
                for (int t = 0; t < dsub; t++) {
                    float diff = sub[t] - c[t];
                    dist += diff * diff;
                }
                if (dist < min_dist) {
                    min_dist = dist;
                    arg = (uint8_t)k;
                }
            }
            codes[i * M + m] = arg;
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* LUT: FR/ops/ascendc/op_kernel/ascendc_ivfpq_subspace_distance.cpp:419-463
 *   ip = sum_j q[j]*cb[j]  (left to right), ip *= -2, dist = (||cb||^2 + ||q_m||^2) + ip.
 * IP metric: lut = ip.  fp16 mode rounds each entry to IEEE half (RNE) and widens again.        */

static void lut_one(const float *q, int d, int M, const float *codebook, int metric, int lut_fp16, float *lut)
{
    int dsub = d / M;
    for (int m = 0; m < M; m++) {
        const float *qm = q + (int64_t)m * dsub;
        float qn = sqnorm(qm, dsub);
        for (int k = 0; k < 256; k++) {
            const float *c = codebook + ((int64_t)m * 256 + k) * dsub;
            float ip = dotp(qm, c, dsub);
            float v;
            if (metric == ORC_METRIC_IP) {
                v = ip;
            } else {
                float cn = sqnorm(c, dsub);
                v = (cn + qn) + (ip * -2.0f);
            }
            if (lut_fp16) {
                v = orc_f16_to_f32(orc_f32_to_f16(v));
            }
            lut[m * 256 + k] = v;
        }
    }
}

ORC_API void orc_lut(const float *q, int64_t nq, int d, int M, const float *codebook, int metric, int lut_fp16,
                     float *lut)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < nq; i++) {
        lut_one(q + i * d, d, M, codebook, metric, lut_fp16, lut + i * (int64_t)M * 256);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* ADC scan: FR/ops/ascendc/op_kernel/ascendc_ivfpq_search_distance_topk.h:39-73
 *   sum_m lut[m*256 + code[m]], accumulated sequentially m = 0..M-1.                           */

static inline float adc_one(const float *lut, const uint8_t *code, int M)
{
    float s = 0.0f;
    for (int m = 0; m < M; m++) {
        s += lut[m * 256 + code[m]];
    }
    return s;
}

ORC_API void orc_adc_list(const float *lut, const uint8_t *codes, int64_t n, int M, float *out)
{
    for (int64_t i = 0; i < n; i++) {
        out[i] = adc_one(lut, codes + i * M, M);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* Full search: FR/ascenddaemon/impl/IndexIVFPQ.cpp:2104-2411 (L1 probe select, L2 LUT,
 * L3 scan + top-k + merge), result padding :2202-2219 / FR/ascend/impl/AscendIndexImpl.cpp:587-650
 * (distance FLT_MAX for L2, label -1; -FLT_MAX for IP as in ..._topk_simt.h:284-293).
 * Candidate order: (distance, probe rank, position in list).
 * Index layout: CSR -- list l owns rows [list_off[l], list_off[l+1]) of codes[.][M] and ids[.].  */

ORC_API void orc_search(int d, int M, int64_t nlist, int metric, const float *cent, const float *codebook,
                        const int64_t *list_off, const uint8_t *codes, const int64_t *ids, const float *q,
                        int64_t nq, int64_t nprobe, int64_t k, int lut_fp16, float *out_dist, int64_t *out_labels,
                        int64_t *out_scanned)
{
    if (nprobe > nlist) {
        nprobe = nlist;
    }
    int64_t *probe = (int64_t *)malloc(sizeof(int64_t) * (size_t)(nq * nprobe));
    orc_coarse_probe(q, nq, cent, nlist, d, metric, nprobe, probe, NULL);
    float pad = metric == ORC_METRIC_IP ? -FLT_MAX : FLT_MAX;
    int64_t scanned_total = 0;
#pragma omp parallel reduction(+ : scanned_total)
    {
        float *lut = (float *)malloc(sizeof(float) * (size_t)M * 256);
        orc_ent *h = (orc_ent *)malloc(sizeof(orc_ent) * (size_t)k);
#pragma omp for schedule(dynamic, 4)
        for (int64_t i = 0; i < nq; i++) {
            lut_one(q + i * d, d, M, codebook, metric, lut_fp16, lut);
            int64_t hn = 0, seq = 0;
            for (int64_t r = 0; r < nprobe; r++) {
                int64_t l = probe[i * nprobe + r];
                int64_t b = list_off[l], e = list_off[l + 1];
                scanned_total += e - b;
                for (int64_t p = b; p < e; p++) {
                    float dist = adc_one(lut, codes + p * M, M);
                    heap_offer(h, &hn, k, dist, seq++, ids[p], metric);
                }
            }
            heap_drain_sorted(h, hn, metric);
            for (int64_t r = 0; r < k; r++) {
                if (r < hn) {
                    out_dist[i * k + r] = h[r].d;
                    out_labels[i * k + r] = h[r].label;
                } else {
                    out_dist[i * k + r] = pad;
                    out_labels[i * k + r] = -1;
                }
            }
        }
        free(lut);
        free(h);
    }
    if (out_scanned) {
        *out_scanned = scanned_total;
    }
    free(probe);
}

/* ------------------------------------------------------------------------------------------ */
/* Flat fp32 (AscendIndexFlat semantics with fp32 distances instead of the reference's fp16:
 * FR/ascendhost/src/index/IndexFlatL2Aicpu.cpp:157-306): same expanded form as the coarse stage,
 * order (distance, position), labels = ids[position] or the position itself.                    */

ORC_API void orc_flat_f32(const float *base, int64_t n, int d, int metric, const int64_t *ids, const float *q,
                          int64_t nq, int64_t k, float *out_dist, int64_t *out_labels)
{
    float *bn = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    orc_sqnorms(base, n, d, bn);
    float pad = metric == ORC_METRIC_IP ? -FLT_MAX : FLT_MAX;
#pragma omp parallel
    {
        orc_ent *h = (orc_ent *)malloc(sizeof(orc_ent) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < nq; i++) {
            const float *qi = q + i * d;
            float qn = sqnorm(qi, d);
            int64_t hn = 0;
            for (int64_t j = 0; j < n; j++) {
                float dj = coarse_one(qi, qn, base + j * d, bn[j], d, metric);
                heap_offer(h, &hn, k, dj, j, ids ? ids[j] : j, metric);
            }
            heap_drain_sorted(h, hn, metric);
            for (int64_t r = 0; r < k; r++) {
                out_dist[i * k + r] = r < hn ? h[r].d : pad;
                out_labels[i * k + r] = r < hn ? h[r].label : -1;
            }
        }
        free(h);
    }
    free(bn);
}

/* ------------------------------------------------------------------------------------------ */
/* Flat int8 L2: integer part of FR/ops/ascendc/op_kernel/ascendc_dist_int8_flat_l2.cpp:201-203,
 * 485-500 (||q||^2 + ||b||^2 - 2 q.b in int32; norms FR/ascenddaemon/impl/IndexInt8Flat.cpp:938-967).
 * The reference's final x scale -> fp16 rounding is NOT applied: distances stay exact int32,
 * order (distance, position).                                                                   */

ORC_API void orc_flat_i8(const int8_t *base, int64_t n, int d, const int64_t *ids, const int8_t *q, int64_t nq,
                         int64_t k, int32_t *out_dist, int64_t *out_labels)
{
    int32_t *bn = (int32_t *)malloc(sizeof(int32_t) * (size_t)(n > 0 ? n : 1));
    for (int64_t j = 0; j < n; j++) {
        int32_t s = 0;
        for (int t = 0; t < d; t++) {
            s += (int32_t)base[j * d + t] * (int32_t)base[j * d + t];
        }
        bn[j] = s;
    }
#pragma omp parallel
    {
        orc_ent *h = (orc_ent *)malloc(sizeof(orc_ent) * (size_t)k);
#pragma omp for schedule(static)
        for (int64_t i = 0; i < nq; i++) {
            const int8_t *qi = q + i * d;
            int32_t qn = 0;
            for (int t = 0; t < d; t++) {
                qn += (int32_t)qi[t] * (int32_t)qi[t];
            }
            int64_t hn = 0;
            for (int64_t j = 0; j < n; j++) {
                int32_t g = 0;
                for (int t = 0; t < d; t++) {
                    g += (int32_t)qi[t] * (int32_t)base[j * d + t];
                }
                int32_t dist = qn + bn[j] - 2 * g;
                /* int32 values up to 512*254^2 < 2^25 are not all exact in float, so keep the
                 * heap key exact by ordering on the integer directly.                          */
                heap_offer(h, &hn, k, (float)0, ((int64_t)dist << 32) | (int64_t)(uint32_t)j, ids ? ids[j] : j,
                           ORC_METRIC_L2);
            }
            heap_drain_sorted(h, hn, ORC_METRIC_L2);
            for (int64_t r = 0; r < k; r++) {
                out_dist[i * k + r] = r < hn ? (int32_t)(h[r].seq >> 32) : INT32_MAX;
                out_labels[i * k + r] = r < hn ? h[r].label : -1;
            }
        }
        free(h);
    }
    free(bn);
}

/* ------------------------------------------------------------------------------------------ */
/* k-means (PARITY UNPINNED: the reference delegates to faiss::Clustering, which is absent).
 * Plain Lloyd; spherical=1 L2-normalises centroids after every update as the reference's
 * training does (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1064-1067, 1170-1172;
 * FR/ascenddaemon/impl/IndexIVFPQ.cpp:508-530).  Initial centroids = rows picked by a seeded
 * Fisher-Yates shuffle.  An empty cluster is re-seeded by splitting the largest one.            */

static uint64_t splitmix(uint64_t *s)
{
    uint64_t z = (*s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

ORC_API double orc_kmeans(const float *x, int64_t n, int d, int64_t kc, int niter, int spherical, uint64_t seed,
                          float *cent)
{
    int64_t *perm = (int64_t *)malloc(sizeof(int64_t) * (size_t)n);
    for (int64_t i = 0; i < n; i++) {
        perm[i] = i;
    }
    uint64_t s = seed;
    for (int64_t i = 0; i < kc && i < n - 1; i++) {
        int64_t j = i + (int64_t)(splitmix(&s) % (uint64_t)(n - i));
        int64_t t = perm[i];
        perm[i] = perm[j];
        perm[j] = t;
    }
    for (int64_t c = 0; c < kc; c++) {
        memcpy(cent + c * d, x + perm[c % n] * d, sizeof(float) * (size_t)d);
    }
    free(perm);
    int64_t *assign = (int64_t *)malloc(sizeof(int64_t) * (size_t)n);
    double *acc = (double *)malloc(sizeof(double) * (size_t)(kc * d));
    int64_t *cnt = (int64_t *)malloc(sizeof(int64_t) * (size_t)kc);
    double obj = 0.0;
    for (int it = 0; it < niter; it++) {
        orc_assign(x, n, cent, kc, d, assign);
        memset(acc, 0, sizeof(double) * (size_t)(kc * d));
        memset(cnt, 0, sizeof(int64_t) * (size_t)kc);
        obj = 0.0;
        for (int64_t i = 0; i < n; i++) {
            int64_t a = assign[i];
            cnt[a]++;
            for (int t = 0; t < d; t++) {
                double df = (double)x[i * d + t] - (double)cent[a * d + t];
                obj += df * df;
                acc[a * d + t] += x[i * d + t];
            }
        }
        for (int64_t c = 0; c < kc; c++) {
            if (cnt[c] > 0) {
                for (int t = 0; t < d; t++) {
                    cent[c * d + t] = (float)(acc[c * d + t] / (double)cnt[c]);
                }
            }
        }
        for (int64_t c = 0; c < kc; c++) {
            if (cnt[c] == 0) {
                int64_t big = 0;
                for (int64_t c2 = 1; c2 < kc; c2++) {
                    if (cnt[c2] > cnt[big]) {
                        big = c2;
                    }
                }
                for (int t = 0; t < d; t++) {
                    float v = cent[big * d + t];
                    float eps = (t & 1) ? 1.0f / 1024 : -1.0f / 1024;
                    cent[c * d + t] = v * (1.0f + eps);
                    cent[big * d + t] = v * (1.0f - eps);
                }
                cnt[c] = cnt[big] / 2;
                cnt[big] -= cnt[c];
            }
        }
        if (spherical) {
            for (int64_t c = 0; c < kc; c++) {
                float nn = sqrtf(sqnorm(cent + c * d, d));
                if (nn > 0.0f) {
                    for (int t = 0; t < d; t++) {
                        cent[c * d + t] /= nn;
                    }
                }
            }
        }
    }
    free(assign);
    free(acc);
    free(cnt);
    return obj;
}

/* Merge of the per-device result lists of one search: FR/ascend/impl/AscendIndexImpl.cpp:587-640.
 * dist/labels: [ndev][n][k], every list best first.  Entries whose label is -1 (or all ones) are
 * skipped wherever they stand; a strict comparison picks the winner, so equal distances go to the
 * lower device; exhausted lists pad with (FLT_MAX, -1) for both metrics. */
ORC_API void orc_merge_results(int ndev, const float *dist, const int64_t *labels, int64_t n, int64_t k, int metric,
                               float *out_dist, int64_t *out_labels)
{
    int64_t *posit = (int64_t *)malloc((size_t)ndev * sizeof(int64_t));
    for (int64_t i = 0; i < n; i++) {
        const int64_t offset = i * k;
        for (int j = 0; j < ndev; j++) {
            posit[j] = 0;
        }
        for (int64_t num = 0; num < k; num++) {
            int id = ndev;
            float best = FLT_MAX;
            int64_t best_label = -1;
            for (int j = 0; j < ndev; j++) {
                const float *dj = dist + (int64_t)j * n * k;
                const int64_t *lj = labels + (int64_t)j * n * k;
                while (posit[j] < k && lj[offset + posit[j]] == -1) {
                    posit[j]++;
                }
                if (posit[j] >= k) {
                    continue;
                }
                const float v = dj[offset + posit[j]];
                const int wins = metric == ORC_METRIC_L2 ? (v < best) : (v > best);
                if (id == ndev || wins) {
                    best = v;
                    best_label = lj[offset + posit[j]];
                    id = j;
                }
            }
            if (id == ndev) {
                out_dist[offset + num] = FLT_MAX;
                out_labels[offset + num] = -1;
            } else {
                out_dist[offset + num] = best;
                out_labels[offset + num] = best_label;
                posit[id]++;
            }
        }
    }
    free(posit);
}

ORC_API int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
