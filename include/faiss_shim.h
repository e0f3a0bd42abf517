// Minimal stand-in for the faiss types that the reference's public classes derive from or exchange data
// with (faiss::Index, MetricType, FaissException, ClusteringParameters, IndexFlat, ProductQuantizer,
// ArrayInvertedLists, IndexIVFPQ): the members copyFrom / copyTo and the class hierarchy touch, under
// faiss 1.10's names.  faiss itself is not a dependency of this build; a project that has faiss defines
// IXA_USE_REAL_FAISS and gets the real headers instead.
#pragma once
#ifdef IXA_USE_REAL_FAISS
#include <faiss/Clustering.h>
#include <faiss/Index.h>
#include <faiss/IndexFlat.h>
#include <faiss/IndexIDMap.h>
#include <faiss/IndexIVFPQ.h>
#include <faiss/IndexScalarQuantizer.h>
#include <faiss/impl/FaissException.h>
#include <faiss/impl/IDSelector.h>
#include <faiss/invlists/InvertedLists.h>
#else
#include <cstddef>
#include <cstdint>
#include <exception>
#include <string>
#include <unordered_set>
#include <vector>

namespace faiss {

using idx_t = int64_t;

enum MetricType { METRIC_INNER_PRODUCT = 0, METRIC_L2 = 1 };

class FaissException : public std::exception {
public:
    explicit FaissException(const std::string &m) : msg(m) {}
    const char *what() const noexcept override { return msg.c_str(); }
    std::string msg;
};

struct SearchParameters {
    virtual ~SearchParameters() {}
};

// The selectors remove_ids takes (faiss/impl/IDSelector.h): a predicate on ids, with the three concrete
// kinds the reference's callers use.
struct IDSelector {
    virtual bool is_member(idx_t id) const = 0;
    virtual ~IDSelector() {}
};
struct IDSelectorRange : IDSelector {
    idx_t imin, imax;   // ids in [imin, imax)
    IDSelectorRange(idx_t imin_, idx_t imax_) : imin(imin_), imax(imax_) {}
    bool is_member(idx_t id) const override { return id >= imin && id < imax; }
};
struct IDSelectorArray : IDSelector {
    size_t n;
    const idx_t *ids;
    IDSelectorArray(size_t n_, const idx_t *ids_) : n(n_), ids(ids_) {}
    bool is_member(idx_t id) const override
    {
        for (size_t i = 0; i < n; i++) {
            if (ids[i] == id) {
                return true;
            }
        }
        return false;
    }
};
struct IDSelectorBatch : IDSelector {
    std::unordered_set<idx_t> set;
    IDSelectorBatch(size_t n, const idx_t *indices) : set(indices, indices + n) {}
    bool is_member(idx_t id) const override { return set.count(id) != 0; }
};

struct ClusteringParameters {
    int niter = 25;
    int nredo = 1;
    bool verbose = false;
    bool spherical = false;
    bool int_centroids = false;
    bool update_index = false;
    bool frozen_centroids = false;
    int min_points_per_centroid = 39;
    int max_points_per_centroid = 256;
    int seed = 1234;
    size_t decode_block_size = 32768;
};

struct Index {
    int d;
    idx_t ntotal = 0;
    bool verbose = false;
    bool is_trained = true;
    MetricType metric_type;
    explicit Index(idx_t d_ = 0, MetricType metric = METRIC_L2) : d((int)d_), metric_type(metric) {}
    virtual ~Index() {}
    virtual void train(idx_t /*n*/, const float * /*x*/) {}
    virtual void add(idx_t n, const float *x) = 0;
    virtual void add_with_ids(idx_t /*n*/, const float * /*x*/, const idx_t * /*xids*/)
    {
        throw FaissException("add_with_ids not implemented for this type of index");
    }
    virtual void search(idx_t n, const float *x, idx_t k, float *distances, idx_t *labels,
                        const SearchParameters *params = nullptr) const = 0;
    virtual void reset() = 0;
    virtual size_t remove_ids(const IDSelector & /*sel*/)
    {
        throw FaissException("remove_ids not implemented for this type of index");
    }
};

// The coarse quantizer of an IndexIVFPQ as copyFrom / copyTo see it: a row store.
struct IndexFlat : Index {
    std::vector<float> xb;
    explicit IndexFlat(idx_t d_ = 0, MetricType metric = METRIC_L2) : Index(d_, metric) {}
    void add(idx_t n, const float *x) override
    {
        xb.insert(xb.end(), x, x + (size_t)n * d);
        ntotal += n;
    }
    void search(idx_t, const float *, idx_t, float *, idx_t *, const SearchParameters * = nullptr) const override
    {
        throw FaissException("the stand-in IndexFlat only stores rows");
    }
    void reset() override
    {
        xb.clear();
        ntotal = 0;
    }
    const float *get_xb() const { return xb.data(); }
};
struct IndexFlatL2 : IndexFlat {
    explicit IndexFlatL2(idx_t d_ = 0) : IndexFlat(d_, METRIC_L2) {}
};
struct IndexFlatIP : IndexFlat {
    explicit IndexFlatIP(idx_t d_ = 0) : IndexFlat(d_, METRIC_INNER_PRODUCT) {}
};

// faiss::IndexScalarQuantizer as the int8 exchange sees it: one byte per dimension in `codes`
// (the reference reads and writes them as int8, FR/ascend/impl/AscendIndexInt8FlatImpl.cpp:414-431, 580-607).
struct IndexScalarQuantizer : Index {
    std::vector<uint8_t> codes;
    size_t code_size = 0;
    explicit IndexScalarQuantizer(idx_t d_ = 0, MetricType metric = METRIC_L2) : Index(d_, metric), code_size((size_t)d_) {}
    void add(idx_t, const float *) override { throw FaissException("the stand-in IndexScalarQuantizer only carries codes"); }
    void search(idx_t, const float *, idx_t, float *, idx_t *, const SearchParameters * = nullptr) const override
    {
        throw FaissException("the stand-in IndexScalarQuantizer only carries codes");
    }
    void reset() override
    {
        codes.clear();
        ntotal = 0;
    }
};

// faiss::IndexIDMap as copyFrom / copyTo see it: an index plus the user ids of its rows.
struct IndexIDMap : Index {
    Index *index = nullptr;
    bool own_fields = false;
    std::vector<idx_t> id_map;
    explicit IndexIDMap(Index *inner = nullptr) : Index(inner ? inner->d : 0, inner ? inner->metric_type : METRIC_L2), index(inner)
    {
        if (inner) {
            ntotal = inner->ntotal;
        }
    }
    ~IndexIDMap() override
    {
        if (own_fields) {
            delete index;
        }
    }
    void add(idx_t, const float *) override { throw FaissException("add does not make sense with IndexIDMap, use add_with_ids"); }
    void add_with_ids(idx_t n, const float *x, const idx_t *xids) override
    {
        index->add(n, x);
        id_map.insert(id_map.end(), xids, xids + n);
        ntotal = index->ntotal;
    }
    void search(idx_t, const float *, idx_t, float *, idx_t *, const SearchParameters * = nullptr) const override
    {
        throw FaissException("the stand-in IndexIDMap only stores rows and ids");
    }
    void reset() override
    {
        index->reset();
        id_map.clear();
        ntotal = 0;
    }
};

struct ProductQuantizer {
    size_t d = 0, M = 0, nbits = 0, dsub = 0, code_size = 0, ksub = 0;
    std::vector<float> centroids;   // [M][ksub][dsub]
    ProductQuantizer() {}
    ProductQuantizer(size_t d_, size_t M_, size_t nbits_) : d(d_), M(M_), nbits(nbits_) { set_derived_values(); }
    void set_derived_values()
    {
        dsub = M ? d / M : 0;
        code_size = (nbits * M + 7) / 8;
        ksub = (size_t)1 << nbits;
        centroids.resize(d * ksub);
    }
};

struct InvertedLists {
    size_t nlist, code_size;
    InvertedLists(size_t nlist_, size_t code_size_) : nlist(nlist_), code_size(code_size_) {}
    virtual ~InvertedLists() {}
    virtual size_t list_size(size_t list_no) const = 0;
    virtual const uint8_t *get_codes(size_t list_no) const = 0;
    virtual const idx_t *get_ids(size_t list_no) const = 0;
    virtual void release_codes(size_t, const uint8_t *) const {}
    virtual void release_ids(size_t, const idx_t *) const {}
    virtual size_t add_entries(size_t list_no, size_t n_entry, const idx_t *ids, const uint8_t *code) = 0;
};

struct ArrayInvertedLists : InvertedLists {
    std::vector<std::vector<uint8_t>> codes;
    std::vector<std::vector<idx_t>> ids;
    ArrayInvertedLists(size_t nlist_, size_t code_size_) : InvertedLists(nlist_, code_size_), codes(nlist_), ids(nlist_) {}
    size_t list_size(size_t l) const override { return ids[l].size(); }
    const uint8_t *get_codes(size_t l) const override { return codes[l].data(); }
    const idx_t *get_ids(size_t l) const override { return ids[l].data(); }
    size_t add_entries(size_t l, size_t n, const idx_t *ids_in, const uint8_t *code) override
    {
        const size_t at = ids[l].size();
        ids[l].insert(ids[l].end(), ids_in, ids_in + n);
        codes[l].insert(codes[l].end(), code, code + n * code_size);
        return at;
    }
};

// faiss::IndexIVFPQ with the members of IndexIVF / Level1Quantizer that the exchange touches.
struct IndexIVFPQ : Index {
    Index *quantizer = nullptr;
    size_t nlist = 0;
    bool own_fields = false;
    ClusteringParameters cp;
    InvertedLists *invlists = nullptr;
    bool own_invlists = false;
    size_t code_size = 0;
    size_t nprobe = 1;
    bool by_residual = true;
    ProductQuantizer pq;
    IndexIVFPQ() {}
    IndexIVFPQ(Index *quantizer_, size_t d_, size_t nlist_, size_t M, size_t nbits_per_idx, MetricType metric = METRIC_L2)
        : Index((idx_t)d_, metric), quantizer(quantizer_), nlist(nlist_), invlists(new ArrayInvertedLists(nlist_, M)),
          own_invlists(true), code_size(M), pq(d_, M, nbits_per_idx)
    {
        is_trained = false;
    }
    ~IndexIVFPQ() override
    {
        if (own_invlists) {
            delete invlists;
        }
        if (own_fields) {
            delete quantizer;
        }
    }
    IndexIVFPQ(const IndexIVFPQ &) = delete;
    IndexIVFPQ &operator=(const IndexIVFPQ &) = delete;
    void replace_invlists(InvertedLists *il, bool own = false)
    {
        if (own_invlists) {
            delete invlists;
        }
        invlists = il;
        own_invlists = own;
    }
    void add(idx_t, const float *) override { throw FaissException("the stand-in IndexIVFPQ only carries data"); }
    void search(idx_t, const float *, idx_t, float *, idx_t *, const SearchParameters * = nullptr) const override
    {
        throw FaissException("the stand-in IndexIVFPQ only carries data");
    }
    void reset() override
    {
        if (invlists) {
            replace_invlists(new ArrayInvertedLists(nlist, code_size), true);
        }
        ntotal = 0;
    }
};

}  // namespace faiss
#endif
