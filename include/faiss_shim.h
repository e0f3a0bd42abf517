// Minimal stand-in for the faiss types that the reference's public classes derive from
// (faiss::Index, faiss::MetricType, faiss::FaissException).  faiss itself is not a dependency of
// this build; a project that already has faiss can define IXA_USE_REAL_FAISS and include the real
// headers instead.
#pragma once
#ifdef IXA_USE_REAL_FAISS
#include <faiss/Index.h>
#include <faiss/impl/FaissException.h>
#else
#include <cstdint>
#include <exception>
#include <string>

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
};

}  // namespace faiss
#endif
