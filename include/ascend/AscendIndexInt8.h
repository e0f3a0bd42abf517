// faiss::ascend::AscendIndexInt8 (FR/ascend/AscendIndexInt8.h:38-110): the root of the int8 index classes
// (not a faiss::Index: its vectors are int8).  Header-only.
#pragma once
#include "AscendIndex.h"

namespace faiss {
namespace ascend {

const int64_t INDEX_INT8_DEFAULT_MEM = 0x2000000;   // 32M

// AscendIndexInt8Config (FR/ascend/AscendIndexInt8.h:38-51)
struct AscendIndexInt8Config {
    inline AscendIndexInt8Config() : deviceList({0}), resourceSize(INDEX_INT8_DEFAULT_MEM) {}
    inline AscendIndexInt8Config(std::initializer_list<int> devices, int64_t resources = INDEX_INT8_DEFAULT_MEM)
        : deviceList(devices), resourceSize(resources)
    {
    }
    inline AscendIndexInt8Config(std::vector<int> devices, int64_t resources = INDEX_INT8_DEFAULT_MEM)
        : deviceList(std::move(devices)), resourceSize(resources)
    {
    }
    std::vector<int> deviceList;
    int64_t resourceSize;
};

class AscendIndexInt8 {
public:
    using idx_t = faiss::idx_t;
    AscendIndexInt8(int dims, faiss::MetricType metric, AscendIndexInt8Config config)
        : d(dims), metric_type(metric), indexConfig(std::move(config))
    {
    }
    virtual ~AscendIndexInt8() {}
    AscendIndexInt8(const AscendIndexInt8 &) = delete;
    AscendIndexInt8 &operator=(const AscendIndexInt8 &) = delete;

    virtual void train(idx_t /*n*/, const int8_t * /*x*/) {}
    void add(idx_t n, const int8_t *x) { add_with_ids(n, x, nullptr); }
    void add(idx_t n, const char *x) { add_with_ids(n, reinterpret_cast<const int8_t *>(x), nullptr); }
    void add_with_ids(idx_t n, const char *x, const idx_t *ids)
    {
        add_with_ids(n, reinterpret_cast<const int8_t *>(x), ids);
    }
    void add_with_ids(idx_t n, const int8_t *x, const idx_t *ids) { addImpl(n, x, ids); }
    void search(idx_t n, const int8_t *x, idx_t k, float *distances, idx_t *labels) const
    {
        searchImpl(n, x, k, distances, labels);
    }
    void search(idx_t n, const char *x, idx_t k, float *distances, idx_t *labels) const
    {
        searchImpl(n, reinterpret_cast<const int8_t *>(x), k, distances, labels);
    }
    // assign (FR/ascend/AscendIndexInt8.h:90): the labels of a search for the k nearest
    void assign(idx_t n, const int8_t *x, idx_t *labels, idx_t k = 1)
    {
        std::vector<float> distances((size_t)n * k);
        searchImpl(n, x, k, distances.data(), labels);
    }
    virtual size_t remove_ids(const faiss::IDSelector & /*sel*/)
    {
        throw faiss::FaissException("remove_ids not implemented for this type of index");
    }
    virtual void reserveMemory(size_t /*numVecs*/) {}
    virtual size_t reclaimMemory() { return 0; }
    std::vector<int> getDeviceList() { return indexConfig.deviceList; }
    int getDim() const { return d; }
    idx_t getNTotal() const { return ntotal; }
    bool isTrained() const { return is_trained; }
    faiss::MetricType getMetricType() const { return metric_type; }

    int d;
    idx_t ntotal = 0;
    bool verbose = false;
    bool is_trained = true;
    faiss::MetricType metric_type;

protected:
    virtual void addImpl(idx_t n, const int8_t *x, const idx_t *ids) = 0;
    virtual void searchImpl(idx_t n, const int8_t *x, idx_t k, float *distances, idx_t *labels) const = 0;
    AscendIndexInt8Config indexConfig;
};

}  // namespace ascend
}  // namespace faiss
