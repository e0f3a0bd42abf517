// extern "C" surface of the library (declared in include/indexsdk_amd.h).  Every entry point
// catches C++ exceptions, stores the message for ixa_last_error() and returns the status code.
#include "../../include/indexsdk_amd.h"

#include <algorithm>
#include <cstring>
#include <memory>
#include <condition_variable>
#include <mutex>
#include <shared_mutex>
#include <type_traits>
#include <new>
#include <string>

#include "flat_index.h"
#include "ivfpq_index.h"
#include "ops.h"
#include "scan.h"

namespace ixa {
void write_faiss_ivfpq(const IvfpqIndex &idx, const char *path);
std::unique_ptr<IvfpqIndex> read_faiss_ivfpq(const char *path, const IvfpqConfig &cfg);
}  // namespace ixa

// Locking follows the reference's MX_INDEX_MULTITHREAD mode (FR/ascend/impl/AscendIndexImpl.h:62, 230;
// AscendIndexImpl.cpp:204, 508-564), always on here: a search takes the handle's lock shared, everything that
// changes the index takes it exclusively.  A search needs a stream and workspaces of its own, so each runs on a
// lane: lane 0 is the index itself, lanes 1..kSearchViews are views that read the index's data in place
// (borrow_from), made on first need.  A search that finds every lane taken waits for one.
template <typename Index>
struct Lanes {
    static constexpr int kSearchViews = 3;
    mutable std::shared_mutex mu;
    mutable std::mutex lane_mu;                       // guards what follows
    mutable std::condition_variable lane_cv;
    mutable std::unique_ptr<Index> views[kSearchViews];
    mutable uint64_t view_version[kSearchViews] = {0, 0, 0};
    mutable uint64_t version = 1;       // counts the calls that may have changed the index
    mutable unsigned busy = 0;          // bit l = lane l is searching
    mutable Index *last = nullptr;      // lane of the search that finished last: "the last search" of the statistics
};

// The IVFPQ handle owns the index through a pointer so that a loader can hand over a finished one.
struct ivfpq_index : Lanes<ixa::IvfpqIndex> {
    std::unique_ptr<ixa::IvfpqIndex> owned;
    ixa::IvfpqIndex &impl;
    ivfpq_index(int d, int metric, int64_t nlist, int M, int nbits, const ixa::IvfpqConfig &c)
        : owned(new ixa::IvfpqIndex(d, metric, nlist, M, nbits, c)), impl(*owned)
    {
        last = owned.get();
    }
    explicit ivfpq_index(std::unique_ptr<ixa::IvfpqIndex> p) : owned(std::move(p)), impl(*owned) { last = owned.get(); }
};

struct flat_index : Lanes<ixa::FlatIndex> {
    ixa::FlatIndex impl;
    flat_index(int d, int metric, int64_t scratch) : impl(d, metric, scratch) { last = &impl; }
};
struct flat_i8_index : Lanes<ixa::FlatI8Index> {
    ixa::FlatI8Index impl;
    flat_i8_index(int d, int metric, int64_t scratch) : impl(d, metric, scratch) { last = &impl; }
};

namespace {

thread_local std::string g_last_error;

template <typename F>
int guarded(F &&f, bool uses_gpu = true)
{
    if (uses_gpu) {
        (void)hipGetLastError();   // an error some earlier caller on this thread left behind is not this call's
    }
    try {
        f();
        return IXA_OK;
    } catch (const ixa::Error &e) {
        g_last_error = e.what();
        return e.code;
    } catch (const std::bad_alloc &) {
        g_last_error = "host allocation failed";
        return IXA_ERR_BAD_ALLOC;
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return IXA_ERR_INNER_ERROR;
    } catch (...) {   // nothing may unwind through a C caller
        g_last_error = "unknown exception";
        return IXA_ERR_INNER_ERROR;
    }
}

ixa::IvfpqIndex *make_view(const ixa::IvfpqIndex &o)
{
    return new ixa::IvfpqIndex(o.d(), o.metric(), o.nlist(), o.M(), 8, o.config());
}
ixa::FlatIndex *make_view(const ixa::FlatIndex &o) { return new ixa::FlatIndex(o.d(), o.metric(), o.scratch_bytes()); }
ixa::FlatI8Index *make_view(const ixa::FlatI8Index &o) { return new ixa::FlatI8Index(o.d(), o.metric(), o.scratch_bytes()); }
// what a view still owes before the data it refers to may move
void settle_view(ixa::IvfpqIndex &v) { v.flush_pending_stats(); }
void settle_view(ixa::FlatIndex &) {}
void settle_view(ixa::FlatI8Index &) {}

// Exclusive use of a handle.  The statistics a view still owes refer to data that the call may move, so they are
// worked out first; a call that may change the index makes every view borrow again.
template <typename H>
struct Exclusive {
    std::unique_lock<std::shared_mutex> lock;
    const H *h;
    bool changes;
    Exclusive(const H *handle, bool may_change) : lock(handle->mu), h(handle), changes(may_change)
    {
        if (changes) {
            for (auto &v : h->views) {
                if (v) {
                    settle_view(*v);
                }
            }
        }
    }
    ~Exclusive()
    {
        if (changes) {
            (void)hipStreamSynchronize(h->impl.stream());   // views read on other streams what this call wrote
            h->version++;
        }
    }
};

// One search on a handle: the lock shared, and a lane for as long as the search runs.
template <typename H>
class SearchLaneOf {
public:
    using Index = std::remove_reference_t<decltype(std::declval<H>().impl)>;
    explicit SearchLaneOf(const H *handle) : shared_(handle->mu), h_(handle)
    {
        std::unique_lock<std::mutex> g(h_->lane_mu);
        const unsigned all = (1u << (1 + H::kSearchViews)) - 1;
        h_->lane_cv.wait(g, [&] { return (h_->busy & all) != all; });
        while (h_->busy >> lane_ & 1u) {
            lane_++;
        }
        if (lane_ > 0) {
            auto &view = h_->views[lane_ - 1];
            if (!view) {
                view.reset(make_view(h_->impl));
            }
            if (h_->view_version[lane_ - 1] != h_->version) {
                view->borrow_from(h_->impl);
                h_->view_version[lane_ - 1] = h_->version;
            }
        }
        h_->busy |= 1u << lane_;
    }
    ~SearchLaneOf()
    {
        {
            std::lock_guard<std::mutex> g(h_->lane_mu);
            h_->busy &= ~(1u << lane_);
            h_->last = &index();
        }
        h_->lane_cv.notify_one();
    }
    SearchLaneOf(const SearchLaneOf &) = delete;
    SearchLaneOf &operator=(const SearchLaneOf &) = delete;
    Index &index() const { return lane_ == 0 ? const_cast<Index &>(h_->impl) : *h_->views[lane_ - 1]; }

private:
    std::shared_lock<std::shared_mutex> shared_;
    const H *h_;
    int lane_ = 0;
};

#define IXA_HANDLE_AS(h, may_change)                                                              \
    IXA_REQUIRE((h) != nullptr, ixa::kErrInvalidParam, "index handle can not be nullptr.");      \
    Exclusive<std::remove_cv_t<std::remove_pointer_t<decltype(h)>>> ixa_handle_lock((h), (may_change))
#define IXA_HANDLE(h) IXA_HANDLE_AS(h, true)        // a call that may change the index
#define IXA_HANDLE_READS(h) IXA_HANDLE_AS(h, false)  // one that only reads it (but uses its stream or workspaces)
#define IXA_SEARCH_LANE(h)                                                                        \
    IXA_REQUIRE((h) != nullptr, ixa::kErrInvalidParam, "index handle can not be nullptr.");      \
    SearchLaneOf<std::remove_cv_t<std::remove_pointer_t<decltype(h)>>> ixa_lane(h)

ixa::IvfpqConfig to_config(const ivfpq_config_t *cfg)
{
    ixa::IvfpqConfig c;
    if (cfg) {
        IXA_REQUIRE(cfg->spherical >= -1 && cfg->spherical <= 1 && cfg->niter >= 0 && cfg->train_samples_per_list >= 1 && cfg->max_train_samples >= 1 &&
                        cfg->scratch_bytes >= (1 << 20) && cfg->code_layout >= -1 && cfg->code_layout <= 2,
                    ixa::kErrInvalidParam, "invalid ivfpq_config_t field");
        c.niter = cfg->niter;
        c.pq_niter = cfg->pq_niter;
        c.spherical = cfg->spherical;
        c.train_samples_per_list = cfg->train_samples_per_list;
        c.max_train_samples = cfg->max_train_samples;
        c.lut_fp16 = cfg->lut_fp16;
        c.code_layout = cfg->code_layout;
        c.scratch_bytes = cfg->scratch_bytes;
        c.seed = cfg->seed;
        c.strict_reference_params = cfg->strict_reference_params;
        c.coarse_bf16 = cfg->coarse_fp32_only ? 0 : 1;
        c.scan_locality = cfg->scan_locality;
        c.coarse_sampled_bound = cfg->coarse_sampled_bound;
        c.pq_spherical = cfg->pq_spherical ? 1 : 0;
        c.coarse_exact_small = cfg->coarse_exact_small;
        c.stage_timings = cfg->stage_timings;
        c.coarse_resident = cfg->coarse_resident ? 1 : 0;
    }
    return c;
}

}  // namespace

extern "C" {

#define IXA_EXPORT __attribute__((visibility("default")))

IXA_EXPORT const char *ixa_last_error(void) { return g_last_error.c_str(); }
IXA_EXPORT const char *ivfpq_last_error(void) { return g_last_error.c_str(); }

IXA_EXPORT void ivfpq_config_default(ivfpq_config_t *cfg)
{
    if (!cfg) {
        return;
    }
    const ixa::IvfpqConfig d;
    std::memset(cfg, 0, sizeof(*cfg));
    cfg->niter = d.niter;
    cfg->pq_niter = d.pq_niter;
    cfg->spherical = d.spherical;
    cfg->train_samples_per_list = d.train_samples_per_list;
    cfg->max_train_samples = d.max_train_samples;
    cfg->lut_fp16 = d.lut_fp16;
    cfg->code_layout = d.code_layout;
    cfg->scratch_bytes = d.scratch_bytes;
    cfg->seed = d.seed;
    cfg->strict_reference_params = d.strict_reference_params;
    cfg->coarse_fp32_only = d.coarse_bf16 ? 0 : 1;
    cfg->scan_locality = d.scan_locality;
    cfg->coarse_sampled_bound = d.coarse_sampled_bound;
    cfg->pq_spherical = d.pq_spherical;
    cfg->coarse_exact_small = d.coarse_exact_small;
    cfg->stage_timings = d.stage_timings;
    cfg->coarse_resident = d.coarse_resident;
}

IXA_EXPORT int ivfpq_create(int d, int metric, int64_t nlist, int msubs, int nbits, const ivfpq_config_t *cfg,
                            ivfpq_index_t **out)
{
    return guarded([&] {
        IXA_REQUIRE(out != nullptr, ixa::kErrInvalidParam, "out can not be nullptr.");
        *out = nullptr;
        const ixa::IvfpqConfig c = to_config(cfg);
        *out = new ivfpq_index(d, metric, nlist, msubs, nbits, c);
    });
}

IXA_EXPORT int ivfpq_last_search_timings(const ivfpq_index_t *h, double *ms_coarse, double *ms_scan)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->last->last_timings(ms_coarse, ms_scan); });
}

IXA_EXPORT int ivfpq_write_faiss(const ivfpq_index_t *h, const char *path)
{
    return guarded([&] { IXA_HANDLE_READS(h); ixa::write_faiss_ivfpq(h->impl, path); });
}

IXA_EXPORT int ivfpq_read_faiss(const char *path, const ivfpq_config_t *cfg, ivfpq_index_t **out)
{
    return guarded([&] {
        IXA_REQUIRE(out != nullptr, ixa::kErrInvalidParam, "out can not be nullptr.");
        *out = nullptr;
        ixa::IvfpqConfig c = to_config(cfg);
        c.strict_reference_params = 0;   // the file decides the shape
        *out = new ivfpq_index(ixa::read_faiss_ivfpq(path, c));
    });
}

IXA_EXPORT int ivfpq_get_shape(const ivfpq_index_t *h, int *d, int *metric, int64_t *nlist, int *msubs)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        if (d) {
            *d = h->impl.d();
        }
        if (metric) {
            *metric = h->impl.metric();
        }
        if (nlist) {
            *nlist = h->impl.nlist();
        }
        if (msubs) {
            *msubs = h->impl.M();
        }
    });
}

IXA_EXPORT int ivfpq_get_code_layout(const ivfpq_index_t *h, int *layout)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        IXA_REQUIRE(layout, ixa::kErrInvalidParam, "layout can not be nullptr.");
        *layout = h->impl.code_layout();
    });
}

IXA_EXPORT int ivfpq_destroy(ivfpq_index_t *h)
{
    return guarded([&] { delete h; });
}

IXA_EXPORT int ivfpq_train(ivfpq_index_t *h, int64_t n, const float *x)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.train(n, x, false); });
}
IXA_EXPORT int ivfpq_train_device(ivfpq_index_t *h, int64_t n, const float *x)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.train(n, x, true); });
}
IXA_EXPORT int ivfpq_set_trained(ivfpq_index_t *h, const float *centroids, const float *codebook)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.set_trained(centroids, codebook); });
}
IXA_EXPORT int ivfpq_get_trained(const ivfpq_index_t *h, float *centroids, float *codebook)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->impl.get_trained(centroids, codebook); });
}
IXA_EXPORT int ivfpq_is_trained(const ivfpq_index_t *h, int *out)
{
    return guarded([&] { IXA_HANDLE_READS(h); IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr."); *out = h->impl.is_trained(); });
}
IXA_EXPORT int ivfpq_add_with_ids(ivfpq_index_t *h, int64_t n, const float *x, const int64_t *ids)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.add(n, x, ids, false); });
}
IXA_EXPORT int ivfpq_add_with_ids_device(ivfpq_index_t *h, int64_t n, const float *x, const int64_t *ids)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.add(n, x, ids, true); });
}
IXA_EXPORT int ivfpq_add_codes(ivfpq_index_t *h, int64_t list, int64_t n, const uint8_t *codes, const int64_t *ids)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.add_codes(list, n, codes, ids); });
}
IXA_EXPORT int ivfpq_set_nprobe(ivfpq_index_t *h, int nprobe)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.set_nprobe(nprobe); });
}
IXA_EXPORT int ivfpq_set_stage_timings(ivfpq_index_t *h, int mode)
{
    return guarded([&] {
        IXA_HANDLE(h);
        IXA_REQUIRE(mode >= -1 && mode <= 1, ixa::kErrInvalidParam, "stage_timings must be -1, 0 or 1");
        h->impl.set_stage_timings(mode);
    });
}
IXA_EXPORT int ivfpq_get_nprobe(const ivfpq_index_t *h, int *out)
{
    return guarded([&] { IXA_HANDLE_READS(h); IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr."); *out = h->impl.nprobe(); });
}
IXA_EXPORT int ivfpq_search(ivfpq_index_t *h, int64_t n, const float *x, int64_t k, float *distances, int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, false); });
}
IXA_EXPORT int ivfpq_search_device(ivfpq_index_t *h, int64_t n, const float *x, int64_t k, float *distances,
                                   int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, true); });
}
IXA_EXPORT int ivfpq_assign(ivfpq_index_t *h, int64_t n, const float *x, int64_t *out)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->impl.assign(n, x, out, false); });
}
IXA_EXPORT int ivfpq_coarse_probe(ivfpq_index_t *h, int64_t n, const float *x, int64_t *out_ids, float *out_dist)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->impl.coarse_probe(n, x, out_ids, out_dist, false); });
}
IXA_EXPORT int ivfpq_encode(ivfpq_index_t *h, int64_t n, const float *x, uint8_t *codes)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->impl.encode(n, x, codes, false); });
}
IXA_EXPORT int ivfpq_list_length(const ivfpq_index_t *h, int64_t list, int64_t *out)
{
    return guarded([&] { IXA_HANDLE_READS(h); IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr."); *out = h->impl.list_length(list); });
}
IXA_EXPORT int ivfpq_get_list(const ivfpq_index_t *h, int64_t list, uint8_t *codes, int64_t *ids)
{
    return guarded([&] { IXA_HANDLE_READS(h); h->impl.get_list(list, codes, ids); });
}
IXA_EXPORT int ivfpq_remove_ids(ivfpq_index_t *h, int64_t n, const int64_t *ids, int64_t *removed)
{
    return guarded([&] {
        IXA_HANDLE(h);
        const int64_t r = h->impl.remove_ids(n, ids);
        if (removed) {
            *removed = r;
        }
    });
}
IXA_EXPORT int ivfpq_remove_range(ivfpq_index_t *h, int64_t imin, int64_t imax, int64_t *removed)
{
    return guarded([&] {
        IXA_HANDLE(h);
        const int64_t r = h->impl.remove_range(imin, imax);
        if (removed) {
            *removed = r;
        }
    });
}
IXA_EXPORT int ivfpq_update(ivfpq_index_t *h, int64_t n, const float *x, const int64_t *ids, int64_t *missing_ids,
                            int64_t *n_missing)
{
    return guarded([&] {
        IXA_HANDLE(h);
        const std::vector<int64_t> m = h->impl.update(n, x, ids);
        if (n_missing) {
            *n_missing = (int64_t)m.size();
        }
        if (missing_ids) {
            std::copy(m.begin(), m.end(), missing_ids);
        }
    });
}
IXA_EXPORT int ivfpq_reserve_memory(ivfpq_index_t *h, int64_t num_vecs)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.reserve_memory(num_vecs); });
}
IXA_EXPORT int ivfpq_reclaim_memory(ivfpq_index_t *h, int64_t *bytes_reclaimed)
{
    return guarded([&] {
        IXA_HANDLE(h);
        const int64_t b = h->impl.reclaim_memory();
        if (bytes_reclaimed) {
            *bytes_reclaimed = b;
        }
    });
}
IXA_EXPORT int ivfpq_arena_state(const ivfpq_index_t *h, int64_t *slots_allocated, int64_t *slots_used,
                                 int64_t *slots_holes)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        int64_t a = 0, u = 0, ho = 0;
        h->impl.arena_state(&a, &u, &ho);
        if (slots_allocated) {
            *slots_allocated = a;
        }
        if (slots_used) {
            *slots_used = u;
        }
        if (slots_holes) {
            *slots_holes = ho;
        }
    });
}
IXA_EXPORT int ivfpq_search_lanes(const ivfpq_index_t *h, int *out)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr.");
        *out = 1;
        for (auto &v : h->views) {
            *out += v ? 1 : 0;
        }
    }, false);
}
IXA_EXPORT int ivfpq_reset(ivfpq_index_t *h)
{
    return guarded([&] { IXA_HANDLE(h); h->impl.reset(); });
}
IXA_EXPORT int ivfpq_ntotal(const ivfpq_index_t *h, int64_t *out)
{
    return guarded([&] { IXA_HANDLE_READS(h); IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr."); *out = h->impl.ntotal(); });
}
IXA_EXPORT int ivfpq_last_search_stats(const ivfpq_index_t *h, ivfpq_search_stats_t *out)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr.");
        const ixa::SearchStats &s = h->last->stats();
        out->scanned_codes = s.scanned_codes;
        out->ms_coarse = s.ms_coarse;
        out->ms_scan = s.ms_scan;
        out->ms_total = s.ms_total;
        out->scan_launches = s.scan_launches;
        out->nsplit = s.nsplit;
        out->scan_waves = s.scan_waves;
        out->shared_pool = s.shared_pool;
        out->coarse_reruns = s.coarse_reruns;
        out->ordered = s.ordered;
        out->coarse_plan = s.coarse_plan;
        out->pages = s.pages;
    });
}

// ---- Flat ---------------------------------------------------------------------------------------

static void copy_stats(const ixa::FlatStats &s, flat_search_stats_t *out)
{
    IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr.");
    out->ms_score = s.ms_score;
    out->ms_select = s.ms_select;
    out->ms_total = s.ms_total;
    out->score_launches = s.score_launches;
    out->exact_reruns = s.exact_reruns;
}

#define IXA_FLAT_COMMON(PFX, HT, ET)                                                                              \
    IXA_EXPORT int PFX##_create(int d, int metric, int64_t scratch_bytes, HT **out)                              \
    {                                                                                                             \
        return guarded([&] {                                                                                      \
            IXA_REQUIRE(out != nullptr, ixa::kErrInvalidParam, "out can not be nullptr.");                        \
            *out = nullptr;                                                                                       \
            *out = new HT(d, metric, scratch_bytes > 0 ? scratch_bytes : ((int64_t)1 << 30));                     \
        });                                                                                                       \
    }                                                                                                             \
    IXA_EXPORT int PFX##_destroy(HT *h) { return guarded([&] { delete h; }); }                                    \
    IXA_EXPORT int PFX##_add_with_ids(HT *h, int64_t n, const ET *x, const int64_t *ids)                         \
    {                                                                                                             \
        return guarded([&] { IXA_HANDLE(h); h->impl.add(n, x, ids, false); });                                    \
    }                                                                                                             \
    IXA_EXPORT int PFX##_add_with_ids_device(HT *h, int64_t n, const ET *x, const int64_t *ids)                  \
    {                                                                                                             \
        return guarded([&] { IXA_HANDLE(h); h->impl.add(n, x, ids, true); });                                     \
    }                                                                                                             \
    IXA_EXPORT int PFX##_get_base(const HT *h, int64_t offset, int64_t n, ET *out)                               \
    {                                                                                                             \
        return guarded([&] { IXA_HANDLE_READS(h); h->impl.get_base(offset, n, out); });                                 \
    }                                                                                                             \
    IXA_EXPORT int PFX##_get_ids(const HT *h, int64_t offset, int64_t n, int64_t *out)                           \
    {                                                                                                             \
        return guarded([&] { IXA_HANDLE_READS(h); h->impl.get_ids(offset, n, out); });                                  \
    }                                                                                                             \
    IXA_EXPORT int PFX##_remove_ids(HT *h, int64_t n, const int64_t *ids, int64_t *removed)                      \
    {                                                                                                             \
        return guarded([&] {                                                                                      \
            IXA_HANDLE(h);                                                                                        \
            const int64_t r = h->impl.remove_ids(n, ids);                                                         \
            if (removed) {                                                                                        \
                *removed = r;                                                                                     \
            }                                                                                                     \
        });                                                                                                       \
    }                                                                                                             \
    IXA_EXPORT int PFX##_remove_range(HT *h, int64_t imin, int64_t imax, int64_t *removed)                       \
    {                                                                                                             \
        return guarded([&] {                                                                                      \
            IXA_HANDLE(h);                                                                                        \
            const int64_t r = h->impl.remove_range(imin, imax);                                                   \
            if (removed) {                                                                                        \
                *removed = r;                                                                                     \
            }                                                                                                     \
        });                                                                                                       \
    }                                                                                                             \
    IXA_EXPORT int PFX##_ntotal(const HT *h, int64_t *out)                                                        \
    {                                                                                                             \
        return guarded([&] {                                                                                      \
            IXA_HANDLE_READS(h);                                                                                  \
            IXA_REQUIRE(out, ixa::kErrInvalidParam, "out can not be nullptr.");                                   \
            *out = h->impl.ntotal();                                                                              \
        });                                                                                                       \
    }                                                                                                             \
    IXA_EXPORT int PFX##_reset(HT *h) { return guarded([&] { IXA_HANDLE(h); h->impl.reset(); }); }                \
    IXA_EXPORT int PFX##_last_search_stats(const HT *h, flat_search_stats_t *out)                                 \
    {                                                                                                             \
        return guarded([&] { IXA_HANDLE_READS(h); copy_stats(h->last->stats(), out); });                                 \
    }

IXA_FLAT_COMMON(flat, flat_index_t, float)
IXA_FLAT_COMMON(flat_i8, flat_i8_index_t, int8_t)

IXA_EXPORT int ixa_merge_search_results(int ndev, int64_t n, int64_t k, int metric, const float *const *dist,
                                        const int64_t *const *labels, float *distances, int64_t *out_labels)
{
    return guarded([&] {
        IXA_REQUIRE(ndev >= 1 && n >= 0 && k >= 1, ixa::kErrInvalidParam, "ndev and k must be >= 1 and n >= 0");
        IXA_REQUIRE(metric == ixa::kMetricL2 || metric == ixa::kMetricInnerProduct, ixa::kErrInvalidParam, "Unsupported metric type");
        IXA_REQUIRE(dist && labels && distances && out_labels, ixa::kErrInvalidParam, "result arrays can not be nullptr.");
        for (int j = 0; j < ndev; j++) {
            IXA_REQUIRE(dist[j] && labels[j], ixa::kErrInvalidParam, "result arrays can not be nullptr.");
        }
        const bool smaller_wins = metric == ixa::kMetricL2;
        std::vector<int64_t> cursor((size_t)ndev);
        for (int64_t q = 0; q < n; q++) {
            const int64_t row = q * k;
            // a cursor always rests on a valid entry of its list, or on k
            auto settle = [&](int j) {
                while (cursor[j] < k && labels[j][row + cursor[j]] == -1) {
                    cursor[j]++;
                }
            };
            for (int j = 0; j < ndev; j++) {
                cursor[j] = 0;
                settle(j);
            }
            for (int64_t out = 0; out < k; out++) {
                int from = -1;
                for (int j = 0; j < ndev; j++) {
                    if (cursor[j] >= k) {
                        continue;
                    }
                    const float v = dist[j][row + cursor[j]];
                    if (from < 0 || (smaller_wins ? v < dist[from][row + cursor[from]] : v > dist[from][row + cursor[from]])) {
                        from = j;
                    }
                }
                if (from < 0) {
                    distances[row + out] = 3.402823466e+38f;
                    out_labels[row + out] = -1;
                    continue;
                }
                distances[row + out] = dist[from][row + cursor[from]];
                out_labels[row + out] = labels[from][row + cursor[from]];
                cursor[from]++;
                settle(from);
            }
        }
    }, false);
}
IXA_EXPORT int ixa_op_distance_flat_l2_mins_fp32(const float *queries_dev, int64_t batch, const float *codes_dev,
                                                 int64_t n, int d, const float *codes_sqr_sum_dev, float *dist_dev,
                                                 float *min_dev, void *stream)
{
    return guarded([&] {
        ixa::op_distance_flat_l2_mins_fp32(queries_dev, batch, codes_dev, n, d, codes_sqr_sum_dev, dist_dev, min_dev,
                                           static_cast<hipStream_t>(stream));
    });
}
IXA_EXPORT int ixa_op_topk_flat_fp32(const float *dists_dev, int64_t batch, int64_t n, int64_t ld, int k, int asc,
                                     float *out_dists_dev, int64_t *out_labels_dev, void *stream)
{
    return guarded([&] {
        IXA_REQUIRE(asc == 1, ixa::kErrInvalidParam, "TopkFlatFp32: only ascending selection (asc = 1) is supported");
        ixa::op_topk_flat_fp32(dists_dev, batch, n, ld, k, out_dists_dev, out_labels_dev, static_cast<hipStream_t>(stream));
    });
}
IXA_EXPORT int ixa_op_ivfpq_subspace_distance(const float *queries_dev, int64_t batch, int d, const float *codebook_dev,
                                              int msubs, int metric, float *lut_dev, void *stream)
{
    return guarded([&] {
        ixa::op_ivfpq_subspace_distance(queries_dev, batch, d, codebook_dev, msubs, metric, lut_dev,
                                        static_cast<hipStream_t>(stream));
    });
}
IXA_EXPORT int ixa_op_ivfpq_search_distance_topk(const float *lut_dev, int64_t batch, int msubs, const uint8_t *code_base_dev,
                                                 const int64_t *code_offset_dev, const int64_t *code_size_dev, int nblocks,
                                                 int k, const int64_t *label_base_dev, const int64_t *label_offset_dev,
                                                 int metric, float *topk_values_dev, int64_t *topk_labels_dev, void *stream)
{
    return guarded([&] {
        ixa::op_ivfpq_search_distance_topk(lut_dev, batch, msubs, code_base_dev, code_offset_dev, code_size_dev, nblocks, k,
                                           label_base_dev, label_offset_dev, metric, topk_values_dev, topk_labels_dev,
                                           static_cast<hipStream_t>(stream));
    });
}
IXA_EXPORT int ixa_op_topk_ivfpq_l3(const int64_t *in_labels_dev, const float *in_values_dev, int tiles, int64_t batch,
                                    int list_k, int k, int asc, float *out_values_dev, int64_t *out_labels_dev, void *stream)
{
    return guarded([&] {
        ixa::op_topk_ivfpq_l3(in_labels_dev, in_values_dev, tiles, batch, list_k, k, asc, out_values_dev, out_labels_dev,
                              static_cast<hipStream_t>(stream));
    });
}
IXA_EXPORT int ivfpq_search_probes_device(ivfpq_index_t *h, int64_t n, const float *x_dev, const int32_t *probes_dev,
                                          int nprobe, int64_t k, float *distances_dev, int64_t *labels_dev)
{
    return guarded([&] {
        IXA_SEARCH_LANE(h);
        ixa_lane.index().search_probes(n, x_dev, probes_dev, nprobe, k, distances_dev, labels_dev);
    });
}
IXA_EXPORT int ivfpq_search_probes_device_noalloc(ivfpq_index_t *h, int64_t n, const float *x_dev,
                                                  const int32_t *probes_dev, int nprobe, int64_t k,
                                                  float *distances_dev, int64_t *labels_dev)
{
    return guarded([&] {
        IXA_HANDLE_READS(h);
        h->impl.search_probes_noalloc(n, x_dev, probes_dev, nprobe, k, distances_dev, labels_dev);
    });
}
IXA_EXPORT int ivfpq_plan_scan_lds(int d, int msubs, int lut_fp16, int code_layout, int nprobe, int nsplit, int k,
                                   int waves, int shared_pool, ivfpq_scan_lds_plan_t *out)
{
    return guarded([&] {
        IXA_REQUIRE(out != nullptr, ixa::kErrInvalidParam, "out can not be nullptr.");
        IXA_REQUIRE(d >= 1 && msubs >= 1 && msubs <= 128 && nprobe >= 1 && nsplit >= 1 && k >= 1 &&
                        (waves == 0 || waves == 4 || waves == 8 || waves == 16) && code_layout >= 0 && code_layout <= 2,
                    ixa::kErrInvalidParam, "invalid scan shape");
        ixa::ScanParams p{};
        int ctl = 0;
        const size_t total = ixa::scan_lds_plan(d, msubs, lut_fp16, code_layout, nprobe, nsplit, k, waves, shared_pool,
                                                &p, &ctl);
        out->waves = p.waves;
        out->shared_pool = p.shared_pool;
        out->cap = p.cap;
        out->merge_n = p.merge_n;
        out->table_n = p.table_n;
        out->off_query = p.off_query;
        out->off_pools = p.off_pools;
        out->off_table = p.off_table;
        out->off_hist = p.off_hist;
        out->off_misc = p.off_misc;
        out->ctl_bytes = ctl;
        out->total_bytes = (int32_t)total;
    }, false);
}
IXA_EXPORT int ixa_copy_probe(const void *src_dev, void *dst_dev, int64_t bytes)
{
    return guarded([&] { ixa::launch_copy_probe(src_dev, dst_dev, bytes); });
}
IXA_EXPORT int ixa_read_probe(const void *src_dev, int64_t bytes, int passes, double *ms_per_pass)
{
    return guarded([&] {
        IXA_REQUIRE(ms_per_pass != nullptr, ixa::kErrInvalidParam, "ms_per_pass can not be nullptr.");
        *ms_per_pass = ixa::launch_read_probe(src_dev, bytes, passes);
    });
}
IXA_EXPORT int flat_search(flat_index_t *h, int64_t n, const float *x, int64_t k, float *distances, int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, false); });
}
IXA_EXPORT int flat_search_with_masks(flat_index_t *h, int64_t n, const float *x, int64_t k, const uint8_t *mask,
                                      float *distances, int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search_with_masks(n, x, k, mask, distances, labels); });
}
IXA_EXPORT int flat_search_device(flat_index_t *h, int64_t n, const float *x, int64_t k, float *distances,
                                  int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, true); });
}
IXA_EXPORT int flat_i8_search(flat_i8_index_t *h, int64_t n, const int8_t *x, int64_t k, int32_t *distances,
                              int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, false); });
}
IXA_EXPORT int flat_i8_search_with_masks(flat_i8_index_t *h, int64_t n, const int8_t *x, int64_t k, const uint8_t *mask,
                                         int32_t *distances, int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search_with_masks(n, x, k, mask, distances, labels); });
}
IXA_EXPORT int flat_i8_search_device(flat_i8_index_t *h, int64_t n, const int8_t *x, int64_t k, int32_t *distances,
                                     int64_t *labels)
{
    return guarded([&] { IXA_SEARCH_LANE(h); ixa_lane.index().search(n, x, k, distances, labels, true); });
}

}  // extern "C"
