// Device-resident IVFPQ index for one MI355X: the counterpart of the reference's per-device
// ascend::IndexIVFPQ (FR/ascenddaemon/impl/IndexIVFPQ.h:47-116, 230-278) together with the host
// orchestration of AscendIndexIVFPQImpl (FR/ascend/impl/AscendIndexIVFPQImpl.cpp).
#pragma once
#include <cstdint>
#include <vector>

#include "common.h"
#include "scan.h"
#include "stream_select.h"

namespace ixa {

struct IvfpqConfig {
    int niter = 25;                   // coarse k-means iterations (reference CPU mode: 25)
    int pq_niter = -1;                // sub-quantizer k-means iterations; -1 = niter (pqNiter)
    int spherical = -1;               // coarse centroids L2-normalised after every update: 1 yes, 0 no, -1 = for inner
                                      // product only (the reference forces it there, AscendIndexIVFPQImpl.cpp:1159-1163;
                                      // its CPU mode also does it for L2, which suits unit-norm data only)
    int pq_spherical = 0;             // 1 = sub-quantizer codewords L2-normalised after every update, as the reference's
                                      // host training does (AscendIndexIVFPQImpl.cpp:1064-1067; its device training does
                                      // not): only sensible when every sub-vector has unit norm
    int train_samples_per_list = 256; // rows sampled per coarse centroid (trainSamplesPerList)
    int64_t max_train_samples = 10000000;  // maxTrainSamples
    int lut_fp16 = 0;                 // LUT entries stored as IEEE half
    int code_layout = -1;             // -1 = pick, 0 = row, 1 = rot32 (M in {32, 64, 96}), 2 = xor48 (M = 48)
    int64_t scratch_bytes = (int64_t)1 << 30;  // budget of the coarse score scratch
    uint64_t seed = 1234;
    int strict_reference_params = 0;  // 1 = enforce the reference's d / nlist / M whitelists
    int scan_locality = -1;           // scan workgroups of large batches ordered by locality: 1, 0, -1 = choose
    int coarse_sampled_bound = -1;    // coarse stage of large batches: 1 / -1 = admission bound from a seed stretch of
                                      // the centroids and a proof by count (no score matrix is written), 0 = the
                                      // whole score matrix of a query block is written and selected from
    int coarse_exact_small = -1;      // a handful of queries (queries x centroids x dims <= 2^27) selects its lists from
                                      // canonical scores of every centroid (two launches, nothing to prove): 1 / -1
                                      // yes, 0 = such batches take the matrix-core plans too
    int stage_timings = -1;           // events around the stages of a search (ms_coarse / ms_scan of the statistics):
                                      // 1 = always, 0 = never, -1 = for pages of 256 queries or more (the three
                                      // event records cost a small batch 5-10 us per call); untimed stages report 0
    int coarse_resident = 1;          // sampled-bound plan: 1 = scores by the resident-query kernel where it has an
                                      // instance (64, 96, 128 dimensions), 0 = by the ring kernel
    int coarse_bf16 = 1;              // 1 = generate coarse candidates with bf16 x 3 matrix products (results
                                      // stay exact: candidates are re-evaluated in fp32 and the superset
                                      // property is verified, with an fp32 rerun if it cannot be proven)
};

struct SearchStats {
    double scanned_codes = 0;   // sum of probed list lengths of the last search
    double ms_coarse = 0;       // stage 1 (scores, selection, refine)
    double ms_scan = 0;         // fused LUT + ADC + top-k kernel (+ merge)
    double ms_total = 0;        // device time of the whole search
    double scan_launches = 0;   // kernel launches the ms_scan figure covers
    double nsplit = 0;
    double scan_waves = 0;
    double shared_pool = 0;
    double coarse_reruns = 0;
    double ordered = 0;
    double coarse_plan = 0;     // 0: score matrix materialised and selected from, 1: sampled bound + proof by count
    double pages = 0;           // query pages the search was served in
};

// Scratch of one scan launch when the caller of scan_params() provides it.
struct ScanScratch {
    int32_t *order;               // 2 n ints: execution order | class of every query
    int32_t *hist;                // 2048 ints, the first 1024 zero on entry: class histogram | cursors
    unsigned long long *partial;  // n * nsplit * k keys (only read when a query is split over workgroups)
};

class IvfpqIndex {
public:
    IvfpqIndex(int d, int metric, int64_t nlist, int M, int nbits, const IvfpqConfig &cfg);
    ~IvfpqIndex();
    IvfpqIndex(const IvfpqIndex &) = delete;
    IvfpqIndex &operator=(const IvfpqIndex &) = delete;

    int d() const { return d_; }
    int M() const { return M_; }
    int metric() const { return metric_; }
    int64_t nlist() const { return nlist_; }
    int64_t ntotal() const { return ntotal_; }
    bool is_trained() const { return trained_; }
    int nprobe() const { return nprobe_; }
    void set_nprobe(int nprobe);
    void set_stage_timings(int mode) { cfg_.stage_timings = mode; }   // as IvfpqConfig::stage_timings, from the next search on
    int code_layout() const { return layout_; }
    hipStream_t stream() const { return stream_; }
    const IvfpqConfig &config() const { return cfg_; }
    // Makes this index a search view of `owner` (same shape and configuration): it reads the owner's trained state
    // and lists in place and searches them on its own stream with its own workspaces, so that searches on the owner
    // and on its views run side by side.  The owner must not change (train, add, remove, reset, set_nprobe ...)
    // while a view is searching, and a view borrows again after every such change before its next search; a view
    // serves searches only.
    void borrow_from(const IvfpqIndex &owner);
    void flush_pending_stats() { flush_stats(); }   // before the lists the statistics refer to change or go away

    // x may live on the host or on the device (on_device says which).
    void train(int64_t n, const float *x, bool on_device);
    void set_trained(const float *centroids, const float *codebook);   // host pointers
    void get_trained(float *centroids, float *codebook) const;          // host pointers, either may be null
    void add(int64_t n, const float *x, const int64_t *ids, bool on_device);
    void add_codes(int64_t list, int64_t n, const uint8_t *codes, const int64_t *ids);  // host pointers
    // n codes for arbitrary lists in one arena rebuild; list order inside a list = input order (host pointers)
    void add_codes_bulk(int64_t n, const int32_t *list_no, const uint8_t *codes, const int64_t *ids);
    void search(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device);
    // stages 2-4 only, on probe lists the caller selected (device pointers)
    void search_probes(int64_t n, const float *x_dev, const int32_t *probes_dev, int nprobe, int64_t k, float *dist_dev,
                       int64_t *labels_dev);
    // search_probes() with every intermediate in the library's static device scratch: no allocation; sizes
    // beyond kNoAllocScratchBytes are refused; leaves the statistics of the last search alone
    void search_probes_noalloc(int64_t n, const float *x_dev, const int32_t *probes_dev, int nprobe, int64_t k,
                               float *dist_dev, int64_t *labels_dev);
    static constexpr size_t kNoAllocScratchBytes = (size_t)8 << 20;
    void assign(int64_t n, const float *x, int64_t *out, bool on_device);               // out: host
    void coarse_probe(int64_t n, const float *x, int64_t *out_ids, float *out_dist, bool on_device);  // out: host
    void encode(int64_t n, const float *x, uint8_t *codes, bool on_device);             // codes: host
    int64_t list_length(int64_t list) const;
    void get_list(int64_t list, uint8_t *codes, int64_t *ids) const;                    // host pointers
    int64_t remove_ids(int64_t n, const int64_t *ids);
    int64_t remove_range(int64_t imin, int64_t imax);   // the ids in [imin, imax)
    void reserve_memory(int64_t num_vecs);   // AscendIndexIVF::reserveMemory
    int64_t reclaim_memory();                // AscendIndexIVF::reclaimMemory: bytes released
    // slots allocated / handed out / abandoned by lists that moved (the arena's fill state)
    void arena_state(int64_t *slots, int64_t *used, int64_t *holes) const
    {
        *slots = arena_slots_;
        *used = arena_used_;
        *holes = hole_slots_;
    }
    // replaces the vectors of ids that exist; returns the ids that do not (host pointers)
    std::vector<int64_t> update(int64_t n, const float *x, const int64_t *ids);
    void reset();
    const SearchStats &stats();   // of the last search; evaluates timings and the scanned-code count on demand
    void last_timings(double *ms_coarse, double *ms_scan);   // device times of the last search only (no device work)

private:
    void check_trained() const;
    void search_page(int64_t n, const float *x, int64_t k, float *dist, int64_t *labels, bool on_device);
    void upload_trained(const float *centroids, const float *codebook);
    void derive_from_centroids();
    // best `nout` lists of every row of device matrix x (canonical arithmetic), device outputs
    void coarse_select(const float *x_dev, int64_t n, int nout, int select_metric, int32_t *out_ids,
                       float *out_dist, bool set_only = false, bool defer_check = false);
    float bf16x3_err_scale(int select_metric) const;
    // redone (may be null): receives the rows that were redone, ascending
    int coarse_finish(const float *x_dev, int nout, int select_metric, int32_t *out_ids, float *out_dist,
                      std::vector<int32_t> *redone = nullptr);
    ScanParams scan_params(const float *xd, int64_t n, const int32_t *probes, int nprobe, int64_t k, float *dd,
                           int64_t *ld, const ScanScratch *ext = nullptr);
    static int scan_nsplit(int64_t n, int nprobe, int64_t k, int64_t codes_per_query);
    void coarse_exact_rows(const float *x_dev, const std::vector<int64_t> &rows, int nout, int select_metric,
                           int32_t *out_ids, float *out_dist);
    void append(int64_t n, const int32_t *list_no_dev, const uint8_t *codes_dev, const int64_t *ids_dev,
                const float *assigned_from = nullptr);
    int64_t remove_sorted_ids(const std::vector<int64_t> &gone, std::vector<uint8_t> *found);
    int64_t remove_selected(const std::vector<int64_t> *gone_ids, int64_t imin, int64_t imax,
                            std::vector<uint8_t> *found);
    void relayout(const std::vector<int32_t> &cap, int64_t min_slots);
    void sync_list_tables();
    void kmeans_coarse(const float *sample_dev, int64_t ns);
    void kmeans_pq(const float *sample_dev, int64_t ns);

    int d_, M_, dsub_, metric_;
    int64_t nlist_;
    IvfpqConfig cfg_;
    int layout_ = 0;
    int nprobe_ = 64;
    bool trained_ = false;
    int64_t ntotal_ = 0;
    hipStream_t stream_ = nullptr;
    hipEvent_t ev_[4] = {nullptr, nullptr, nullptr, nullptr};

    DeviceBuffer<float> centroids_, cnorm_, codebook_, cbnorm_;
    DeviceBuffer<uint16_t> centroids_split_, ws_xsplit_;   // bf16 x 3 splits (candidate generation only)
    DeviceBuffer<uint8_t> centroids_tiled_;                // centroids_split_ in matrix-core order (flat_i8.h), or empty
    DeviceBuffer<float> cnorm_pad_;                        // [norms | zeros], each padded to whole tiles with +inf
    DeviceBuffer<int32_t> ws_flag_;
    DeviceBuffer<int32_t> ws_redo_;                    // rows of the queries a search scans a second time
    DeviceBuffer<int32_t> ws_order_, ws_order_hist_;   // execution order of the scan (heaviest queries first)
    int32_t max_list_len_ = 0;
    int last_coarse_reruns_ = 0;
    int last_coarse_plan_ = 0;        // plan of the last coarse_select(): 0 materialised, 1 sampled bound
    bool last_coarse_exact_ = false;  // the last coarse_select() selected from canonical scores: nothing to verify
    int64_t last_coarse_n_ = 0;       // its number of queries
    bool sampled_bound_ok_ = true;    // cleared when the sampled bound failed too many proofs on this index
    bool flag_pending_ = true;   // ws_flag_[0] may be non-zero: clear it before the next coarse stage
    bool stats_pending_ = false;
    bool stats_timed_ = false;   // the last search recorded its stage events
    int64_t stats_rows_ = 0;
    int stats_nprobe_ = 0;
    // the probe lists and list lengths the pending statistics refer to are about to change
    void flush_stats()
    {
        if (stats_pending_) {
            stats();
        }
    }
    float cmax_ = 0.f;                                      // largest centroid norm
    int dp_ = 0;                                            // d rounded up to a multiple of 32
    // arena
    DeviceBuffer<uint8_t> codes_;
    DeviceBuffer<int64_t> ids_;
    DeviceBuffer<int64_t> list_off_dev_;
    DeviceBuffer<int32_t> list_len_dev_;
    std::vector<int64_t> list_off_;   // first slot of each list (host mirror)
    std::vector<int32_t> list_len_;   // its valid entries
    std::vector<int32_t> list_cap_;   // the slots it owns (a multiple of 64, >= its length)
    std::vector<int32_t> touch_mark_; // scratch of append(): -1, or the list's place among the touched lists
    std::vector<int32_t> add_pos_;    // scratch of append(): position of every new vector inside its list
    PinnedBuffer add_stage_, add_pack_;   // append(): assignments coming down, kernel inputs going up
    PinnedBuffer io_stage_;               // host searches: queries going up, results coming down
    DeviceBuffer<int64_t> ws_add_pack_, ws_add_ids_;
    DeviceBuffer<int32_t> ws_add_lists_;
    DeviceBuffer<uint8_t> ws_add_codes_;
    int64_t arena_slots_ = 0;         // slots allocated
    int64_t arena_used_ = 0;          // slots handed out so far (lists and holes)
    int64_t hole_slots_ = 0;          // slots inside the used part that no list owns any more
    // search workspaces (grown on demand, reused between calls)
    DeviceBuffer<float> ws_x_, ws_qn_, ws_dist_, ws_exact_;
    StreamSelectWorkspace<float> ws_sel_;
    DeviceBuffer<unsigned long long> ws_running_;
    DeviceBuffer<int32_t> ws_cand_, ws_probes_;
    DeviceBuffer<int64_t> ws_labels_;
    DeviceBuffer<unsigned long long> ws_partial_, ws_counter_;
    SearchStats stats_;
};

}  // namespace ixa
