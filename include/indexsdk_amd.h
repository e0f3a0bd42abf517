/*
 * C ABI of the MI355X-native IVFPQ / Flat search path.
 *
 * This is the drop-in boundary for the search hot path of Ascend IndexSDK's Faiss-style
 * AscendIndexIVFPQ / AscendIndexFlat / AscendIndexInt8Flat classes: plain pointers and sizes,
 * no C++ or framework types.  Each entry point names the reference interface it stands in for
 * (paths relative to the reference root; FR/ = feature_retrieval/src/ascendfaiss/).
 *
 * Conventions
 *   - every function returns an int status: 0 = ok, otherwise a code with the numeric values of
 *     the reference's APP_ERROR enum (FR/common/ErrorCode.h:26-73); ixa_last_error() returns the
 *     message of the last failure on the calling thread.  The reference's public layer turns such
 *     codes into faiss::FaissException; the C++ wrappers in include/ascend do the same.
 *   - host pointers are caller-owned, row-major, no alignment requirement; outputs are
 *     pre-allocated by the caller (n * k elements), as in faiss::Index::search.
 *   - the *_device variants take DEVICE pointers (16-byte aligned, row-major) and leave their
 *     results in device memory; they synchronise the index's stream before returning.
 *   - metric: 0 = inner product, 1 = L2 (faiss::MetricType values).
 *   - missing results: label -1, distance FLT_MAX for L2 and -FLT_MAX for inner product
 *     (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2202-2219; FR/ascend/impl/AscendIndexImpl.cpp:587-650).
 *   - every handle may be used from several threads.  A handle locks as the reference does under
 *     MX_INDEX_MULTITHREAD (FR/ascend/impl/AscendIndexImpl.h:62, 230; AscendIndexImpl.cpp:204, 508-564): the
 *     searches (ivfpq_search, ivfpq_search_device, ivfpq_search_probes_device; flat_search, flat_search_device,
 *     flat_search_with_masks and their flat_i8_ forms) take the lock shared and up to four of them run side by
 *     side, each on a stream and workspaces of its own; every other call takes it exclusively.  Different
 *     handles never wait for each other.
 *   - there is no CPU fallback: every entry point fails with IXA_ERR_INDEX_NOT_INIT when no
 *     HIP device is present.
 */
#ifndef INDEXSDK_AMD_H
#define INDEXSDK_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IXA_OK 0
#define IXA_ERR_BAD_ALLOC 1001        /* APP_ERR_ACL_BAD_ALLOC */
#define IXA_ERR_OP_EXEC_FAILED 1017   /* APP_ERR_ACL_OP_EXEC_FAILED */
#define IXA_ERR_INVALID_PARAM 2001    /* APP_ERR_INVALID_PARAM */
#define IXA_ERR_NOT_IMPLEMENT 2008    /* APP_ERR_NOT_IMPLEMENT */
#define IXA_ERR_ILLEGAL_OPERATION 2009
#define IXA_ERR_INNER_ERROR 2010      /* APP_ERR_INNER_ERROR */
#define IXA_ERR_INDEX_NOT_INIT 2016   /* APP_ERR_INDEX_NOT_INIT */

#define IXA_METRIC_INNER_PRODUCT 0
#define IXA_METRIC_L2 1

/* Message of the last failed call on this thread ("" if none). */
const char *ixa_last_error(void);
/* The same string under the index family's prefix. */
const char *ivfpq_last_error(void);

/* Copies bytes (a multiple of 16) between two DEVICE buffers with a plain copy kernel and waits for
 * it.  No counterpart in the reference: it is the kernel of known size that hardware traffic
 * counters (FETCH_SIZE / WRITE_SIZE) of the search kernels are scaled by. */
int ixa_copy_probe(const void *src_dev, void *dst_dev, int64_t bytes);
/* Reads bytes (a multiple of 16) of a DEVICE buffer `passes` times with a plain streaming kernel (16 bytes
 * per lane and step, grid-stride) and returns the average duration of a pass in *ms_per_pass: the rate
 * at which this GPU's memory system delivers a sequential read, the practical ceiling that the scan
 * kernel's achieved bytes per second are to be read against (the published peak is not reachable by
 * any kernel).  The buffer should be several times larger than the last-level cache.  No counterpart in
 * the reference. */
int ixa_read_probe(const void *src_dev, int64_t bytes, int passes, double *ms_per_pass);

/* AscendIndexImpl::mergeSearchResult  FR/ascend/impl/AscendIndexImpl.cpp:587-640: merges the result
 * lists that `ndev` devices (or index shards) returned for the same n queries into one list of k per
 * query.  dist[j] / labels[j]: HOST arrays [n][k] of device j, best first.  Entries with label -1 are
 * skipped wherever they stand, equal distances go to the lower j, and lists that run out are padded
 * with (FLT_MAX, -1).  Host code, as in the reference; touches no GPU. */
int ixa_merge_search_results(int ndev, int64_t n, int64_t k, int metric, const float *const *dist,
                             const int64_t *const *labels, float *distances, int64_t *out_labels);

/* ---------------------------------------------------------------------------------------------
 * Stage operators.  The reference runs the search path as named device operators through
 * AscendOperator::exec(inputs, outputs, stream) (FR/ascenddaemon/utils/AscendOperator.cpp:33-45,
 * 110-121; descriptors FR/ascenddaemon/impl/IndexIVFPQ.cpp:1633-1755).  The entry points below take the
 * same tensors as plain DEVICE pointers, allocate nothing, and only queue work on `stream` (a
 * hipStream_t, NULL = the null stream): a host layer that keeps the reference's staging can call them
 * where it called exec.  Arithmetic: the reference's scalar order (left to right, no FMA).
 * ------------------------------------------------------------------------------------------- */

/* Operator "DistanceFlatL2MinsAtFP32" (FR/ops/ascendc/op_kernel/distance_flat_l2_mins_at_fp32.cpp:95-251).
 * inputs: queries [batch][d], codes [n][d], codesSqrSum [n];  outputs: dist [batch][n] =
 * (|q|^2 + codesSqrSum[j]) - g - g, and min [batch][ceil(n/64)*2] (may be NULL): per burst of 64 codes
 * the smallest distance followed by its position in the burst (uint32 bit pattern), as WholeReduceMin
 * leaves them.  The operator's third output (a completion flag for the AICPU top-k that polls it) has
 * no counterpart: stream order does that job here. */
int ixa_op_distance_flat_l2_mins_fp32(const float *queries_dev, int64_t batch, const float *codes_dev, int64_t n,
                                      int d, const float *codes_sqr_sum_dev, float *dist_dev, float *min_dev,
                                      void *stream);

/* Operator "TopkFlatFp32" (FR/ops/cpukernel/impl/topk_flat_fp32_cpu_kernel.cpp:223-384) as the IVFPQ
 * path uses it (attrs asc = 1, k = nprobe, one block, one page; IndexIVFPQ.cpp:2127-2136).
 * input: dists [batch][ld], the first n columns of a row are valid;  outputs: outdists [batch][k]
 * ascending and outlabel [batch][k] (column numbers, int64), padded with (FLT_MAX, -1) when n < k.
 * Equal distances go to the lower column (the reference's heap leaves that order unspecified).
 * k <= 2048; asc must be 1. */
int ixa_op_topk_flat_fp32(const float *dists_dev, int64_t batch, int64_t n, int64_t ld, int k, int asc,
                          float *out_dists_dev, int64_t *out_labels_dev, void *stream);

/* Operator "AscendcIvfpqSubspaceDistance" (FR/ops/ascendc/op_kernel/ascendc_ivfpq_subspace_distance.cpp:
 * 197-477).  inputs: queries [batch][d], codeBook [msubs][256][d/msubs];  output: lut [batch][msubs][256]
 * = (|cb|^2 + |q_m|^2) + (-2 q_m.cb) for IXA_METRIC_L2, q_m.cb for IXA_METRIC_INNER_PRODUCT. */
int ixa_op_ivfpq_subspace_distance(const float *queries_dev, int64_t batch, int d, const float *codebook_dev,
                                   int msubs, int metric, float *lut_dev, void *stream);

/* Operator "AscendcIvfpqSearchDistanceL2" (descriptor FR/ascenddaemon/impl/IndexIVFPQ.cpp:1706-1755, kernel
 * FR/ops/ascendc/op_kernel/ascendc_ivfpq_search_distance_topk.h:39-93, 556-810) with the reference's operands:
 * queryPQ = lut [batch][msubs][256] (what ixa_op_ivfpq_subspace_distance wrote); codeBase + codeOffset
 * [batch][nblocks] (byte offsets of the code blocks a query scans) + codeSize [batch][nblocks] (valid codes of
 * each, 0 = skip; at most 262144, the reference's block size); labelBase + labelOffset [batch][nblocks]
 * (element offsets of the blocks' ids).  Codes are row-major, msubs bytes each.  Outputs = the operator's
 * topkIndexFinal / topkValueFinal: the k best (label, distance) per query, best first, padded with -1 and
 * FLT_MAX (-FLT_MAX for IXA_METRIC_INNER_PRODUCT, where lut holds inner products and larger is better).  The
 * operator's per-block intermediates (distResult, topkIndex, topkValue, flag) stay inside the launch.
 * k <= 384 (the reference: 320), nblocks <= 2048. */
int ixa_op_ivfpq_search_distance_topk(const float *lut_dev, int64_t batch, int msubs, const uint8_t *code_base_dev,
                                      const int64_t *code_offset_dev, const int64_t *code_size_dev, int nblocks, int k,
                                      const int64_t *label_base_dev, const int64_t *label_offset_dev, int metric,
                                      float *topk_values_dev, int64_t *topk_labels_dev, void *stream);
/* Operator "TopkIvfpqL3" (descriptor FR/ascenddaemon/impl/IndexIVFPQ.cpp:1844-1877, kernel
 * FR/ops/cpukernel/impl/topk_ivfpq_l3_cpu_kernel.cpp:176-250): merges the best-first lists of `tiles` launches
 * of the operator above, in_labels / in_values [tiles][batch][list_k] (label -1 = padding), into the k best per
 * query.  asc = 1: smaller is better (L2); 0: larger is better.  tiles x list_k <= 16384. */
int ixa_op_topk_ivfpq_l3(const int64_t *in_labels_dev, const float *in_values_dev, int tiles, int64_t batch, int list_k,
                         int k, int asc, float *out_values_dev, int64_t *out_labels_dev, void *stream);

/* ---------------------------------------------------------------------------------------------
 * IVFPQ
 * ------------------------------------------------------------------------------------------- */

typedef struct ivfpq_index ivfpq_index_t;

/* Mirrors AscendIndexIVFPQConfig / AscendIndexIVFConfig (FR/ascend/AscendIndexIVFPQ.h:32-68,
 * FR/ascend/AscendIndexIVF.h:37-72); fields that only make sense on Ascend hardware (deviceList,
 * useDistributedCoarse, enableQueryParallelSearch) have no counterpart on one GPU. */
typedef struct ivfpq_config {
    int32_t niter;                  /* cp.niter of the coarse k-means; reference CPU mode uses 25 */
    int32_t pq_niter;               /* pqNiter; -1 = niter */
    int32_t spherical;              /* cp.spherical for the COARSE quantizer: 1 = centroids L2-normalised after every
                                       update, 0 = plain Lloyd, -1 (default) = normalised for inner product only.  The
                                       reference forces it for inner product and, in its CPU mode, for L2 as well
                                       (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1159-1171), which suits unit-norm data
                                       only.  Sub-quantizer codebooks: see pq_spherical.  useKmeansPP of the reference's config selects WHERE it
                                       trains (its NPU k-means or faiss on the host); this build always trains on the
                                       device, seeded with random samples, whatever that flag says. */
    int32_t train_samples_per_list; /* trainSamplesPerList */
    int64_t max_train_samples;      /* maxTrainSamples */
    int32_t lut_fp16;               /* 1 = store the per-query LUT as IEEE half (accumulate in fp32) */
    int32_t code_layout;            /* -1 = choose (by measurement: rotated for 64 and 96 sub-quantizers and for 32
                                       with a half LUT, xor-rotated for 48 with an fp32 LUT, else row-major),
                                       0 = row-major codes, 1 = bank-rotated (M in {32,64,96}),
                                       2 = xor-rotated (M = 48, fp32 LUT) */
    int64_t scratch_bytes;          /* resourceSize: bound of the coarse-score scratch in HBM */
    uint64_t seed;                  /* sampling / initialisation seed */
    int32_t strict_reference_params;/* 1 = enforce the reference whitelists d in {128}, nlist in
                                       {1024..16384, 262144, 524288}, M in {2,4,8,16,32} */
    int32_t coarse_fp32_only;       /* 0 = coarse candidates from bf16 x 3 matrix products, re-evaluated in fp32 and
                                       verified (results identical to the fp32 plan); 1 = fp32 matrix products only */
    int32_t scan_locality;          /* execution order of the scan's workgroups in large batches (results do not
                                       depend on it): 1 = queries that probe the same lists run side by side on one
                                       XCD, 0 = input order, -1 = choose */
    int32_t coarse_sampled_bound;   /* coarse stage of large batches (results do not depend on it): 1 or -1 = the
                                       admission bound of the score kernel comes from a seed stretch of the centroids
                                       and every query's candidate list is proven complete by count, so that no
                                       query x centroid score matrix is written; 0 = the score matrix of a query
                                       block is written and selected from */
    int32_t pq_spherical;           /* 1 = sub-quantizer codewords L2-normalised after every update, as the
                                       reference's host training does (faiss Clustering with cp.spherical = true,
                                       FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1064-1067); 0 (default) = plain Lloyd,
                                       as its device training */
    int32_t coarse_exact_small;     /* coarse stage of a handful of queries (queries x centroids x dims <= 2^27;
                                       results do not depend on it): 1 or -1 = the probed lists are selected from
                                       canonical scores of every centroid (two small launches, exact by
                                       construction), 0 = such batches go through the matrix-core plans and their
                                       proof as well */
    int32_t stage_timings;          /* HIP events around the stages of a search, which ms_coarse / ms_scan / ms_total
                                       of ivfpq_last_search_stats come from: 1 = always, 0 = never, -1 (default) =
                                       for pages of 256 queries or more (recording them costs a small batch 5-10 us
                                       per call); a search without them reports 0 ms */
    int32_t coarse_resident;        /* score launches of the sampled-bound coarse plan (results do not depend on it):
                                       1 (default) = by the kernel that keeps a tile of queries resident in LDS and
                                       reads the centroids from matrix-core order, where it has an instance (64, 96
                                       and 128 dimensions); 0 = by the ring kernel that streams both operands */
} ivfpq_config_t;

/* Fills *cfg with the defaults. */
void ivfpq_config_default(ivfpq_config_t *cfg);

/* AscendIndexIVFPQ(dims, metric, nlist, msubs, nbits, config)  FR/ascend/AscendIndexIVFPQ.h:74-75;
 * parameter checks and messages of checkParams, FR/ascend/impl/AscendIndexIVFPQImpl.cpp:510-525.
 * cfg may be NULL. */
int ivfpq_create(int d, int metric, int64_t nlist, int msubs, int nbits, const ivfpq_config_t *cfg,
                 ivfpq_index_t **out);
/* ~AscendIndexIVFPQ */
int ivfpq_destroy(ivfpq_index_t *h);

/* AscendIndexIVFPQ::train(n, x)  FR/ascend/impl/AscendIndexIVFPQImpl.cpp:1144-1252 */
int ivfpq_train(ivfpq_index_t *h, int64_t n, const float *x);
int ivfpq_train_device(ivfpq_index_t *h, int64_t n, const float *x_dev);

/* Stands in for copyFrom(const faiss::IndexIVFPQ*) (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:392-425):
 * injects trained quantizers.  centroids[nlist*d], codebook[msubs*256*dsub] laid out like
 * faiss pq.centroids.  Codes added later are computed on the RAW vector (by_residual = false). */
int ivfpq_set_trained(ivfpq_index_t *h, const float *centroids, const float *codebook);
/* Stands in for copyTo(faiss::IndexIVFPQ*) (:453-508), quantizer part; either output may be NULL. */
int ivfpq_get_trained(const ivfpq_index_t *h, float *centroids, float *codebook);
int ivfpq_is_trained(const ivfpq_index_t *h, int *out);

/* File form of copyTo / copyFrom(faiss::IndexIVFPQ*) (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:392-508): the
 * index is written / read in the byte layout of faiss::write_index for an IndexIVFPQ with an IndexFlat
 * coarse quantizer, by_residual = false and ArrayInvertedLists (fourcc "IwPQ"), so that faiss::read_index
 * on the CPU side opens the file and files written by faiss::write_index load here.  Reading rejects
 * by_residual = true (the reference accepts it silently and returns wrong distances).  cfg may be NULL. */
int ivfpq_write_faiss(const ivfpq_index_t *h, const char *path);
int ivfpq_read_faiss(const char *path, const ivfpq_config_t *cfg, ivfpq_index_t **out);
/* Shape of an index (the public members d, metric_type, nlist and pq.M of the reference class); any output
 * may be NULL. */
int ivfpq_get_shape(const ivfpq_index_t *h, int *d, int *metric, int64_t *nlist, int *msubs);
/* The code layout in use (the values of ivfpq_config_t.code_layout, never -1). */
int ivfpq_get_code_layout(const ivfpq_index_t *h, int *layout);

/* AscendIndex::add / add_with_ids  FR/ascend/AscendIndex.h:66-71, AscendIndexIVFPQImpl.cpp:694-864.
 * ids == NULL numbers the vectors ntotal, ntotal+1, ... */
int ivfpq_add_with_ids(ivfpq_index_t *h, int64_t n, const float *x, const int64_t *ids);
int ivfpq_add_with_ids_device(ivfpq_index_t *h, int64_t n, const float *x_dev, const int64_t *ids_dev);
/* ascend::IndexIVFPQ::addPQCodes(listId, n, codes, ids)  FR/ascenddaemon/impl/IndexIVFPQ.cpp:210-235;
 * codes row-major [n][msubs]. */
int ivfpq_add_codes(ivfpq_index_t *h, int64_t list, int64_t n, const uint8_t *codes, const int64_t *ids);

/* AscendIndexIVF::setNumProbes / getNumProbes  FR/ascend/AscendIndexIVF.h:96-99.  nprobe >= 1; a value above
 * the number of lists is clamped to it; more than 2048 probed lists are refused. */
int ivfpq_set_nprobe(ivfpq_index_t *h, int nprobe);
int ivfpq_get_nprobe(const ivfpq_index_t *h, int *out);
/* config.stage_timings of an existing index, from its next search on (-1, 0 or 1).  No counterpart in the
 * reference: a serving loop of small batches switches the stage events off, a measurement switches them on. */
int ivfpq_set_stage_timings(ivfpq_index_t *h, int mode);

/* AscendIndex::search(n, x, k, distances, labels)  FR/ascend/AscendIndex.h:79-80 ->
 * ascend::IndexIVFPQ::searchImpl  FR/ascenddaemon/impl/IndexIVFPQ.cpp:2373-2411.  0 < n < 1e9, 0 < k <= 2048
 * (the reference's device limit is 320); with 128 sub-quantizers and an fp32 LUT, k <= 1024.  A batch whose
 * per-query workspaces would exceed config.scratch_bytes is served page by page (AscendIndexImpl::searchPaged,
 * FR/ascend/impl/AscendIndexImpl.cpp:296-346); the results do not depend on the paging. */
int ivfpq_search(ivfpq_index_t *h, int64_t n, const float *x, int64_t k, float *distances, int64_t *labels);
int ivfpq_search_device(ivfpq_index_t *h, int64_t n, const float *x_dev, int64_t k, float *distances_dev,
                        int64_t *labels_dev);
/* Stages 2-4 only, on probe lists the caller selected: operators "AscendcIvfpqSearchDistanceL2" +
 * "TopkIvfpqL3" (IndexIVFPQ::searchImplL3, FR/ascenddaemon/impl/IndexIVFPQ.cpp:2162-2347), the LUT being
 * built inside the launch.  probes_dev: [n][nprobe] list ids (int32, DEVICE); -1, like any other value
 * outside [0, nlist), means no list; a list named twice is scanned twice.  Results as ivfpq_search_device.  Waits for the results.
 * ivfpq_last_search_stats afterwards reports the plan of the scan only (no stage timings are taken here). */
int ivfpq_search_probes_device(ivfpq_index_t *h, int64_t n, const float *x_dev, const int32_t *probes_dev, int nprobe,
                               int64_t k, float *distances_dev, int64_t *labels_dev);

/* ivfpq_search_probes_device for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference.  It runs on the index's own stream and waits
 * for the results, so it is not meant to be called under stream capture.  Same
 * arguments, same results bit for bit; it calls no hipMalloc / hipFree: the intermediates of the launch
 * (sanitised probe lists, execution order, split partials) lie in a static device array of
 * IVFPQ_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends.  A call that
 * needs more (8192 + 8 n + 4 n nprobe + 8 n nsplit k bytes, each term rounded up to 256; nsplit <= 64 is
 * the number of workgroups a query of a small batch is split over) fails with IXA_ERR_INVALID_PARAM and a
 * message that names the need and the limit.  All calls on one GPU share the array; inside one process
 * they take turns (a lock), and the array's contents mean nothing between calls.  It leaves
 * ivfpq_last_search_stats alone.  Waits for the results. */
#define IVFPQ_NOALLOC_SCRATCH_BYTES (8u << 20)
int ivfpq_search_probes_device_noalloc(ivfpq_index_t *h, int64_t n, const float *x_dev, const int32_t *probes_dev,
                                       int nprobe, int64_t k, float *distances_dev, int64_t *labels_dev);

/* Coarse assignment used by add (nearest centroid under L2), FR/ascend/impl/AscendIndexIVFPQImpl.cpp:603-672;
 * out[n]. */
int ivfpq_assign(ivfpq_index_t *h, int64_t n, const float *x, int64_t *out_list_ids);
/* L1 level of search: the nprobe best lists per query, best first
 * (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2104-2164); out_ids[n*nprobe], out_dist may be NULL. */
int ivfpq_coarse_probe(ivfpq_index_t *h, int64_t n, const float *x, int64_t *out_ids, float *out_dist);
/* Host PQ encoder of the reference (AscendIndexIVFPQImpl.cpp:879-921) on the device; codes[n][msubs]. */
int ivfpq_encode(ivfpq_index_t *h, int64_t n, const float *x, uint8_t *codes);

/* AscendIndexIVF::getListLength / getListCodesAndIds  FR/ascend/AscendIndexIVF.h:108-111;
 * codes[len*msubs] row-major, ids[len]; either may be NULL. */
int ivfpq_list_length(const ivfpq_index_t *h, int64_t list, int64_t *out);
int ivfpq_get_list(const ivfpq_index_t *h, int64_t list, uint8_t *codes, int64_t *ids);

/* AscendIndexIVFPQ::remove_ids(n, ids)  FR/ascend/AscendIndexIVFPQ.h:90; *removed may be NULL. */
int ivfpq_remove_ids(ivfpq_index_t *h, int64_t n, const int64_t *ids, int64_t *removed);
/* AscendIndex::remove_ids(IDSelectorRange)  FR/ascend/AscendIndex.h:78 -> AscendIndexIVFImpl::removeImpl
 * (FR/ascend/impl/AscendIndexIVFImpl.cpp:432-440): the vectors whose id lies in [imin, imax) leave; lists keep
 * the order of their survivors, as with ivfpq_remove_ids. */
int ivfpq_remove_range(ivfpq_index_t *h, int64_t imin, int64_t imax, int64_t *removed);
/* AscendIndexIVFPQ::update(n, x, ids)  FR/ascend/AscendIndexIVFPQ.h:92, AscendIndexIVFPQImpl.cpp:540-601:
 * vectors whose id exists are replaced (delete + add); ids that do not exist are written to
 * missing_ids (room for n entries, may be NULL) and counted in *n_missing (may be NULL). */
int ivfpq_update(ivfpq_index_t *h, int64_t n, const float *x, const int64_t *ids, int64_t *missing_ids,
                 int64_t *n_missing);
/* AscendIndexIVF::reserveMemory(numVecs)  FR/ascend/AscendIndexIVF.h:101-102: makes room for num_vecs more vectors, so
 * that adding them does not replace the code arena (lists still move inside it as they outgrow their slack). */
int ivfpq_reserve_memory(ivfpq_index_t *h, int64_t num_vecs);
/* AscendIndexIVF::reclaimMemory()  FR/ascend/AscendIndexIVF.h:104-106: shrinks the code arena to what the lists hold
 * (their slack and the holes moved lists left are given back); *bytes_reclaimed may be NULL. */
int ivfpq_reclaim_memory(ivfpq_index_t *h, int64_t *bytes_reclaimed);
/* Fill state of the code arena, in slots of msubs + 8 bytes: allocated, handed out to lists (their slack included)
 * or abandoned, and abandoned by lists that moved.  Any output may be NULL.  No counterpart in the reference
 * (whose lists are separate device vectors): a diagnostic of the amortised add path. */
int ivfpq_arena_state(const ivfpq_index_t *h, int64_t *slots_allocated, int64_t *slots_used, int64_t *slots_holes);
/* How many search lanes (streams with workspaces of their own) the handle has made so far: 1, plus one for every
 * further search that was ever in flight at the same time, up to 4.  No counterpart in the reference: a diagnostic of
 * the shared search lock. */
int ivfpq_search_lanes(const ivfpq_index_t *h, int *out);
/* AscendIndexIVF::reset()  FR/ascend/AscendIndexIVF.h:93: drops the lists, keeps the quantizers. */
int ivfpq_reset(ivfpq_index_t *h);
int ivfpq_ntotal(const ivfpq_index_t *h, int64_t *out);

/* LDS plan of the fused LUT + scan + top-k kernel for a shape, as the launcher lays it out: byte offsets of the
 * regions the kernel addresses inside its dynamic LDS, and the total.  Host code only (no GPU is touched; it
 * works without one): what a test holds against the regions' sizes to prove that no region ends outside the
 * allocation.  waves = 0 asks for the plan the launcher would choose; 4, 8 or 16 with shared_pool 0 / 1 for
 * the layout of that workgroup size and pool kind.  No counterpart in the reference. */
typedef struct ivfpq_scan_lds_plan {
    int32_t waves, shared_pool; /* wavefronts per workgroup; 1 = one workgroup-wide candidate pool */
    int32_t cap;                /* keys per pool */
    int32_t merge_n;            /* keys of the pool region (waves x cap private pools, or cap) */
    int32_t table_n;            /* probed lists per workgroup */
    int32_t off_query, off_pools, off_table, off_hist, off_misc; /* the LUT starts at 0 */
    int32_t ctl_bytes;          /* control block of the shared pool, at off_misc + 8 x waves */
    int32_t total_bytes;
} ivfpq_scan_lds_plan_t;
int ivfpq_plan_scan_lds(int d, int msubs, int lut_fp16, int code_layout, int nprobe, int nsplit, int k, int waves,
                        int shared_pool, ivfpq_scan_lds_plan_t *out);

/* Device timings of the last ivfpq_search* call, measured with HIP events on the index's stream (0 for a
 * search that recorded none: config.stage_timings).  No counterpart in the reference (it prints std::chrono
 * timers when verbose). */
typedef struct ivfpq_search_stats {
    double scanned_codes; /* sum of the lengths of all probed lists */
    double ms_coarse;     /* stage 1: scores + selection + refine */
    double ms_scan;       /* fused LUT + ADC scan + top-k (+ merge kernel when nsplit > 1) */
    double ms_total;
    double scan_launches; /* kernel launches covered by ms_scan */
    double nsplit;        /* workgroups per query in the scan */
    double scan_waves;    /* wavefronts per scan workgroup */
    double shared_pool;   /* 1: one workgroup-wide candidate pool (large k), 0: one pool per wavefront */
    double coarse_reruns; /* queries whose matrix-core coarse result could not be proven complete and that were
                             redone from canonical scores of all centroids */
    double ordered;       /* 1: the scan started its queries in order of decreasing work (few, heavy workgroups),
                             2: in locality order */
    double coarse_plan;   /* 0: the coarse stage wrote the score matrix and selected from it, 1: sampled bound +
                             proof by count (queries without proof are part of coarse_reruns) */
    double pages;         /* query pages the search was served in (more than one: the sums of the pages' times,
                             scanned codes and reruns are reported; the plan fields are the last page's) */
} ivfpq_search_stats_t;
int ivfpq_last_search_stats(const ivfpq_index_t *h, ivfpq_search_stats_t *out);
/* Device times of the last search only (HIP events on the index's stream, in ms; 0 for a search that recorded
 * none: config.stage_timings); either output may be NULL.
 * Unlike ivfpq_last_search_stats, which counts the scanned codes with a kernel launch and a host
 * synchronisation the first time it is called after a search, this call does no device work, so it can sit
 * inside a timed loop.  No counterpart in the reference: a measurement aid. */
int ivfpq_last_search_timings(const ivfpq_index_t *h, double *ms_coarse, double *ms_scan);

/* ---------------------------------------------------------------------------------------------
 * Flat (brute force): the coarse stage in isolation
 * ------------------------------------------------------------------------------------------- */

typedef struct flat_index flat_index_t;       /* fp32 vectors, L2 or inner product */
typedef struct flat_i8_index flat_i8_index_t; /* int8 vectors, exact int32 L2 */

typedef struct flat_search_stats {
    double ms_score;       /* fp32: all score + selection launches of the last search */
    double ms_select;      /* fp32: exact refine + label mapping */
    double ms_total;
    double score_launches; /* number of (query block, base chunk) score launches */
    double exact_reruns;   /* fp32: queries whose candidate list could not be proven complete and that were
                              redone from canonical scores of the whole base */
} flat_search_stats_t;

/* AscendIndexFlat(dims, metric, config)  FR/ascend/AscendIndexFlat.h:48-90.  scratch_bytes bounds the
 * score scratch in HBM (the role of config.resourceSize); 0 = default (1 GiB).
 * Distances are fp32 in the canonical expanded form (the reference returns fp16-rounded values:
 * FR/ascend/impl/AscendIndexFlatImpl.cpp:444-446). */
int flat_create(int d, int metric, int64_t scratch_bytes, flat_index_t **out);
int flat_destroy(flat_index_t *h);
/* AscendIndex::add / add_with_ids  FR/ascend/AscendIndex.h:66-71; ids == NULL numbers from ntotal. */
int flat_add_with_ids(flat_index_t *h, int64_t n, const float *x, const int64_t *ids);
int flat_add_with_ids_device(flat_index_t *h, int64_t n, const float *x_dev, const int64_t *ids_dev);
/* AscendIndex::search  FR/ascend/AscendIndex.h:79-80 -> IndexFlatL2Aicpu::searchImpl
 * (FR/ascendhost/src/index/IndexFlatL2Aicpu.cpp:157-306). */
int flat_search(flat_index_t *h, int64_t n, const float *x, int64_t k, float *distances, int64_t *labels);
int flat_search_device(flat_index_t *h, int64_t n, const float *x_dev, int64_t k, float *distances_dev,
                       int64_t *labels_dev);
/* AscendIndexFlat::search_with_masks  FR/ascend/AscendIndexFlat.h:78-82 (FR/ascend/impl/AscendIndexFlatImpl.cpp:461-511):
 * mask = n rows of ceil(ntotal / 8) bytes in host memory; query i may only return the vectors whose bit is
 * set in row i (the vector at storage position p: bit p % 8 of byte p / 8).  Results as flat_search on the
 * vectors that take part; fewer than k of them leave (FLT_MAX | -FLT_MAX, -1).  Every stretch of the score
 * matrix is written and masked before the selection reads it, so this is slower than flat_search. */
int flat_search_with_masks(flat_index_t *h, int64_t n, const float *x, int64_t k, const uint8_t *mask, float *distances,
                           int64_t *labels);
/* AscendIndexFlat::getBase / getBaseSize  FR/ascend/AscendIndexFlat.h; rows [offset, offset + n). */
int flat_get_base(const flat_index_t *h, int64_t offset, int64_t n, float *out);
int flat_get_ids(const flat_index_t *h, int64_t offset, int64_t n, int64_t *out);
int flat_ntotal(const flat_index_t *h, int64_t *out);
/* AscendIndex::remove_ids(const faiss::IDSelector &)  FR/ascend/AscendIndex.h:78 -> AscendIndexImpl::removeImpl
 * (FR/ascend/impl/AscendIndexImpl.cpp:208-270) + Index::removeIdsBatch (FR/ascenddaemon/impl/Index.cpp:86-113):
 * the vectors whose id is one of the n ids (IDSelectorBatch; ids the index does not hold and repeats are
 * ignored) or lies in [imin, imax) (IDSelectorRange) leave the index; *removed (may be NULL) = how many.
 * As in the reference every removed position, from the highest to the lowest, is refilled with the vector
 * that is last at that moment, so the order of the remaining vectors (getBase / getIdxMap) is the reference's. */
int flat_remove_ids(flat_index_t *h, int64_t n, const int64_t *ids, int64_t *removed);
int flat_remove_range(flat_index_t *h, int64_t imin, int64_t imax, int64_t *removed);
int flat_reset(flat_index_t *h);
int flat_last_search_stats(const flat_index_t *h, flat_search_stats_t *out);

/* AscendIndexInt8Flat(dims, metric, config)  FR/ascend/AscendIndexInt8.h:53-96 (L2 only here).
 * Distances are the exact int32 values |q|^2 + |b|^2 - 2 q.b; the reference multiplies by
 * 0.01 / min(d/64, max(d/128 + 1, 4)) and rounds to fp16
 * (FR/ops/ascendc/op_kernel/ascendc_dist_int8_flat_l2.cpp:201-203, 491-500), which is not done here.
 * Ties on distance resolve to the vector added first. */
int flat_i8_create(int d, int metric, int64_t scratch_bytes, flat_i8_index_t **out);
int flat_i8_destroy(flat_i8_index_t *h);
int flat_i8_add_with_ids(flat_i8_index_t *h, int64_t n, const int8_t *x, const int64_t *ids);
int flat_i8_add_with_ids_device(flat_i8_index_t *h, int64_t n, const int8_t *x_dev, const int64_t *ids_dev);
/* AscendIndexInt8::search(n, const int8_t *x, k, distances, labels)  FR/ascend/AscendIndexInt8.h:70-72 */
int flat_i8_search(flat_i8_index_t *h, int64_t n, const int8_t *x, int64_t k, int32_t *distances, int64_t *labels);
int flat_i8_search_device(flat_i8_index_t *h, int64_t n, const int8_t *x_dev, int64_t k, int32_t *distances_dev,
                          int64_t *labels_dev);
/* AscendIndexInt8Flat::search_with_masks  FR/ascend/AscendIndexInt8Flat.h:98-99; as flat_search_with_masks
 * (missing results: distance INT32_MAX, label -1). */
int flat_i8_search_with_masks(flat_i8_index_t *h, int64_t n, const int8_t *x, int64_t k, const uint8_t *mask,
                              int32_t *distances, int64_t *labels);
int flat_i8_get_base(const flat_i8_index_t *h, int64_t offset, int64_t n, int8_t *out);
/* AscendIndexInt8Flat::getIdxMap  FR/ascend/AscendIndexInt8Flat.h:83 */
int flat_i8_get_ids(const flat_i8_index_t *h, int64_t offset, int64_t n, int64_t *out);
int flat_i8_ntotal(const flat_i8_index_t *h, int64_t *out);
/* AscendIndexInt8::remove_ids(const faiss::IDSelector &)  FR/ascend/AscendIndexInt8.h:88 ->
 * AscendIndexInt8FlatImpl::removeImpl (FR/ascend/impl/AscendIndexInt8FlatImpl.cpp:819-867); as flat_remove_*. */
int flat_i8_remove_ids(flat_i8_index_t *h, int64_t n, const int64_t *ids, int64_t *removed);
int flat_i8_remove_range(flat_i8_index_t *h, int64_t imin, int64_t imax, int64_t *removed);
int flat_i8_reset(flat_i8_index_t *h);
int flat_i8_last_search_stats(const flat_i8_index_t *h, flat_search_stats_t *out);

#ifdef __cplusplus
}
#endif
#endif /* INDEXSDK_AMD_H */
