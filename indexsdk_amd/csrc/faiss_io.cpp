// Interchange with faiss: an IVFPQ index is written and read in the byte layout of
// faiss::write_index / read_index for a faiss::IndexIVFPQ (faiss 1.10, impl/index_write.cpp):
//
//   u32 "IwPQ"
//   index header:  i32 d, i64 ntotal, i64 1<<20, i64 1<<20, u8 is_trained, i32 metric_type (0 = IP, 1 = L2)
//   u64 nlist, u64 nprobe
//   quantizer:     u32 "IxF2" | "IxFI", index header (ntotal = nlist), u64 nlist*d, f32 centroids[nlist*d]
//   direct map:    u8 0 (none), u64 0 (empty array)
//   u8 by_residual (must be 0), u64 code_size (= M)
//   product quantizer: u64 d, u64 M, u64 nbits (8), u64 M*256*dsub, f32 centroids[M][256][dsub]
//   inverted lists: u32 "ilar", u64 nlist, u64 code_size, u32 "full" + u64 nlist + u64 sizes[nlist]
//                   (or u32 "sprs" + u64 2*n + (list, size) pairs when at most half the lists are
//                   non-empty), then for every non-empty list: u8 codes[n*code_size], i64 ids[n]
//
// It is the file form of what the reference moves in copyFrom / copyTo
// (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:392-508).  Unlike the reference, reading REJECTS an index
// built with by_residual = true: its codes encode residuals, which this search path cannot serve.
#include <cstdio>
#include <cstring>
#include <memory>
#include <vector>

#include "ivfpq_index.h"

namespace ixa {

namespace {

constexpr uint32_t fourcc(const char (&s)[5])
{
    return (uint32_t)(unsigned char)s[0] | ((uint32_t)(unsigned char)s[1] << 8) |
           ((uint32_t)(unsigned char)s[2] << 16) | ((uint32_t)(unsigned char)s[3] << 24);
}

struct File {
    FILE *f = nullptr;
    const char *path;
    File(const char *p, const char *mode) : path(p)
    {
        IXA_REQUIRE(p != nullptr, kErrInvalidParam, "path can not be nullptr.");
        f = std::fopen(p, mode);
        IXA_REQUIRE(f != nullptr, kErrInvalidParam, "cannot open %s", p);
    }
    ~File()
    {
        if (f) {
            std::fclose(f);
        }
    }
    void put(const void *p, size_t bytes)
    {
        IXA_REQUIRE(bytes == 0 || std::fwrite(p, 1, bytes, f) == bytes, kErrInner, "write to %s failed", path);
    }
    void get(void *p, size_t bytes)
    {
        IXA_REQUIRE(bytes == 0 || std::fread(p, 1, bytes, f) == bytes, kErrInvalidParam, "%s is truncated", path);
    }
    template <typename T>
    void put1(T v)
    {
        put(&v, sizeof(T));
    }
    template <typename T>
    T get1()
    {
        T v;
        get(&v, sizeof(T));
        return v;
    }
};

void put_header(File &f, int d, int64_t ntotal, bool trained, int metric)
{
    f.put1<int32_t>(d);
    f.put1<int64_t>(ntotal);
    f.put1<int64_t>((int64_t)1 << 20);
    f.put1<int64_t>((int64_t)1 << 20);
    f.put1<uint8_t>(trained ? 1 : 0);
    f.put1<int32_t>(metric == kMetricL2 ? 1 : 0);
}

struct Header {
    int d;
    int64_t ntotal;
    bool trained;
    int metric;
};

Header get_header(File &f)
{
    Header h;
    h.d = f.get1<int32_t>();
    h.ntotal = f.get1<int64_t>();
    f.get1<int64_t>();
    f.get1<int64_t>();
    h.trained = f.get1<uint8_t>() != 0;
    const int32_t mt = f.get1<int32_t>();
    IXA_REQUIRE(mt == 0 || mt == 1, kErrInvalidParam, "%s: metric_type %d is not supported (0 = IP, 1 = L2)", f.path, mt);
    h.metric = mt == 1 ? kMetricL2 : kMetricInnerProduct;
    return h;
}

}  // namespace

void write_faiss_ivfpq(const IvfpqIndex &idx, const char *path)
{
    IXA_REQUIRE(idx.is_trained(), kErrIndexNotInit, "index is not trained");
    File f(path, "wb");
    const int d = idx.d(), M = idx.M();
    const int64_t nlist = idx.nlist();
    std::vector<float> cent((size_t)nlist * d), cb((size_t)256 * d);
    idx.get_trained(cent.data(), cb.data());

    f.put1<uint32_t>(fourcc("IwPQ"));
    put_header(f, d, idx.ntotal(), true, idx.metric());
    f.put1<uint64_t>((uint64_t)nlist);
    f.put1<uint64_t>((uint64_t)idx.nprobe());
    f.put1<uint32_t>(idx.metric() == kMetricL2 ? fourcc("IxF2") : fourcc("IxFI"));
    put_header(f, d, nlist, true, idx.metric());
    f.put1<uint64_t>(cent.size());
    f.put(cent.data(), cent.size() * sizeof(float));
    f.put1<uint8_t>(0);
    f.put1<uint64_t>(0);
    f.put1<uint8_t>(0);   // by_residual
    f.put1<uint64_t>((uint64_t)M);
    f.put1<uint64_t>((uint64_t)d);
    f.put1<uint64_t>((uint64_t)M);
    f.put1<uint64_t>(8);
    f.put1<uint64_t>(cb.size());
    f.put(cb.data(), cb.size() * sizeof(float));

    f.put1<uint32_t>(fourcc("ilar"));
    f.put1<uint64_t>((uint64_t)nlist);
    f.put1<uint64_t>((uint64_t)M);
    std::vector<uint64_t> sizes((size_t)nlist);
    int64_t non_empty = 0;
    for (int64_t l = 0; l < nlist; l++) {
        sizes[(size_t)l] = (uint64_t)idx.list_length(l);
        non_empty += sizes[(size_t)l] > 0;
    }
    if (non_empty > nlist / 2) {
        f.put1<uint32_t>(fourcc("full"));
        f.put1<uint64_t>(sizes.size());
        f.put(sizes.data(), sizes.size() * 8);
    } else {
        std::vector<uint64_t> pairs;
        for (int64_t l = 0; l < nlist; l++) {
            if (sizes[(size_t)l] > 0) {
                pairs.push_back((uint64_t)l);
                pairs.push_back(sizes[(size_t)l]);
            }
        }
        f.put1<uint32_t>(fourcc("sprs"));
        f.put1<uint64_t>(pairs.size());
        f.put(pairs.data(), pairs.size() * 8);
    }
    std::vector<uint8_t> codes;
    std::vector<int64_t> ids;
    for (int64_t l = 0; l < nlist; l++) {
        const size_t n = (size_t)sizes[(size_t)l];
        if (n == 0) {
            continue;
        }
        codes.resize(n * M);
        ids.resize(n);
        idx.get_list(l, codes.data(), ids.data());
        f.put(codes.data(), codes.size());
        f.put(ids.data(), ids.size() * 8);
    }
}

std::unique_ptr<IvfpqIndex> read_faiss_ivfpq(const char *path, const IvfpqConfig &cfg)
{
    File f(path, "rb");
    // every size the file states is held against the index's limits and against the file's own length before
    // anything is allocated, cast or divided by it
    IXA_REQUIRE(std::fseek(f.f, 0, SEEK_END) == 0, kErrInvalidParam, "%s: can not seek", path);
    const long file_len = std::ftell(f.f);
    IXA_REQUIRE(file_len >= 0 && std::fseek(f.f, 0, SEEK_SET) == 0, kErrInvalidParam, "%s: can not seek", path);
    const uint64_t file_bytes = (uint64_t)file_len;
    IXA_REQUIRE(f.get1<uint32_t>() == fourcc("IwPQ"), kErrInvalidParam, "%s is not a faiss IndexIVFPQ file (IwPQ)", path);
    const Header h = get_header(f);
    const uint64_t nlist = f.get1<uint64_t>(), nprobe = f.get1<uint64_t>();
    IXA_REQUIRE(h.d >= 1 && h.d <= 4096 && nlist >= 1 && nlist <= ((uint64_t)1 << 20) && h.ntotal >= 0 &&
                    (h.metric == kMetricL2 || h.metric == kMetricInnerProduct),
                kErrInvalidParam, "%s: d = %d, nlist = %lu, ntotal = %ld or metric = %d is outside what an index holds", path,
                h.d, (unsigned long)nlist, (long)h.ntotal, h.metric);
    IXA_REQUIRE(nlist * (uint64_t)h.d * 4 <= file_bytes, kErrInvalidParam, "%s is shorter than its coarse quantizer", path);
    const uint32_t q4 = f.get1<uint32_t>();
    IXA_REQUIRE(q4 == fourcc("IxF2") || q4 == fourcc("IxFI"), kErrInvalidParam,
                "%s: the coarse quantizer must be an IndexFlat (IxF2 / IxFI)", path);
    const Header qh = get_header(f);
    const uint64_t nfloat = f.get1<uint64_t>();
    IXA_REQUIRE(qh.d == h.d && (uint64_t)qh.ntotal == nlist && nfloat == nlist * (uint64_t)h.d, kErrInvalidParam,
                "%s: coarse quantizer holds %lu floats, expected nlist * d = %lu", path, (unsigned long)nfloat,
                (unsigned long)(nlist * (uint64_t)h.d));
    std::vector<float> cent((size_t)nfloat);
    f.get(cent.data(), cent.size() * sizeof(float));
    const uint8_t map_type = f.get1<uint8_t>();
    const uint64_t map_n = f.get1<uint64_t>();
    IXA_REQUIRE(map_type != 2, kErrInvalidParam, "%s: hashtable direct maps are not supported", path);
    if (map_n) {
        IXA_REQUIRE(map_n <= file_bytes / 8 && std::fseek(f.f, (long)(map_n * 8), SEEK_CUR) == 0, kErrInvalidParam,
                    "%s is truncated (direct map of %lu entries)", path, (unsigned long)map_n);
    }
    const uint8_t by_residual = f.get1<uint8_t>();
    IXA_REQUIRE(by_residual == 0, kErrInvalidParam,
                "%s was built with by_residual = true: its codes encode residuals and cannot be searched here", path);
    const uint64_t code_size = f.get1<uint64_t>();
    const uint64_t pq_d = f.get1<uint64_t>(), M = f.get1<uint64_t>(), nbits = f.get1<uint64_t>();
    IXA_REQUIRE(pq_d == (uint64_t)h.d && nbits == 8 && M >= 1 && M <= 128 && code_size == M &&
                    (uint64_t)h.d % M == 0, kErrInvalidParam,
                "%s: product quantizer d=%lu M=%lu nbits=%lu code_size=%lu is not supported", path, (unsigned long)pq_d,
                (unsigned long)M, (unsigned long)nbits, (unsigned long)code_size);
    const uint64_t ncb = f.get1<uint64_t>();
    IXA_REQUIRE(ncb == (uint64_t)256 * h.d, kErrInvalidParam, "%s: codebook holds %lu floats, expected %lu", path,
                (unsigned long)ncb, (unsigned long)(256 * (uint64_t)h.d));
    std::vector<float> cb((size_t)ncb);
    f.get(cb.data(), cb.size() * sizeof(float));

    auto idx = std::make_unique<IvfpqIndex>(h.d, h.metric, (int64_t)nlist, (int)M, 8, cfg);
    idx->set_trained(cent.data(), cb.data());
    idx->set_nprobe((int)std::min<uint64_t>(std::max<uint64_t>(nprobe, 1), nlist));

    const uint32_t il = f.get1<uint32_t>();
    if (il == fourcc("il00")) {
        return idx;
    }
    IXA_REQUIRE(il == fourcc("ilar"), kErrInvalidParam, "%s: only ArrayInvertedLists (ilar) are supported", path);
    const uint64_t il_nlist = f.get1<uint64_t>(), il_cs = f.get1<uint64_t>();
    IXA_REQUIRE(il_nlist == nlist && il_cs == code_size, kErrInvalidParam, "%s: inverted lists do not match the index", path);
    std::vector<uint64_t> sizes((size_t)nlist, 0);
    const uint32_t lt = f.get1<uint32_t>();
    const uint64_t nv = f.get1<uint64_t>();
    if (lt == fourcc("full")) {
        IXA_REQUIRE(nv == nlist, kErrInvalidParam, "%s: list size table has %lu entries", path, (unsigned long)nv);
        f.get(sizes.data(), sizes.size() * 8);
    } else {
        IXA_REQUIRE(lt == fourcc("sprs") && nv % 2 == 0 && nv <= 2 * nlist, kErrInvalidParam, "%s: bad list size table", path);
        std::vector<uint64_t> pairs((size_t)nv);
        f.get(pairs.data(), pairs.size() * 8);
        for (size_t i = 0; i < pairs.size(); i += 2) {
            IXA_REQUIRE(pairs[i] < nlist, kErrInvalidParam, "%s: list number out of range", path);
            sizes[(size_t)pairs[i]] = pairs[i + 1];
        }
    }
    // lists are appended in pages of a few million codes: one arena rebuild per page
    constexpr size_t kPage = (size_t)4 << 20;
    std::vector<int32_t> list_no;
    std::vector<uint8_t> codes;
    std::vector<int64_t> ids;
    auto flush = [&]() {
        if (!list_no.empty()) {
            idx->add_codes_bulk((int64_t)list_no.size(), list_no.data(), codes.data(), ids.data());
            list_no.clear();
            codes.clear();
            ids.clear();
        }
    };
    uint64_t total = 0;
    for (uint64_t l = 0; l < nlist; l++) {
        const size_t n = (size_t)sizes[(size_t)l];
        if (n == 0) {
            continue;
        }
        IXA_REQUIRE(n < ((uint64_t)1 << 31) && (uint64_t)n * (M + 8) <= file_bytes, kErrInvalidParam,
                    "%s: list %lu is longer than the file", path, (unsigned long)l);
        const size_t at = list_no.size();
        list_no.resize(at + n, (int32_t)l);
        codes.resize((at + n) * M);
        ids.resize(at + n);
        f.get(codes.data() + at * M, n * M);
        f.get(ids.data() + at, n * 8);
        total += n;
        if (list_no.size() >= kPage) {
            flush();
        }
    }
    flush();
    IXA_REQUIRE((int64_t)total == h.ntotal, kErrInvalidParam, "%s: lists hold %lu vectors, header says %ld", path,
                (unsigned long)total, (long)h.ntotal);
    return idx;
}

}  // namespace ixa
