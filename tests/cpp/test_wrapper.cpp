// Host-side check of the C++ wrappers: constructor validation messages as in
// FR/ut/TestAscendIndexUTIVFPQ.cpp:77-184.  With a GPU present (argv[1] == "gpu") it also runs a
// tiny train/add/search through the class interface.
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "ascend/AscendIndexFlat.h"
#include "ascend/AscendIndexIVFPQ.h"

using namespace faiss::ascend;

static int failures = 0;
#define EXPECT(cond)                                                   \
    do {                                                               \
        if (!(cond)) {                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            failures++;                                                \
        }                                                              \
    } while (0)

static std::string construct_msg(int dim, int nlist, int msub, int nbit)
{
    try {
        AscendIndexIVFPQConfig conf({0});
        AscendIndexIVFPQ index(dim, faiss::METRIC_L2, nlist, msub, nbit, conf);
    } catch (std::exception &e) {
        return e.what();
    }
    return "";
}

int main(int argc, char **argv)
{
    EXPECT(construct_msg(64, 1024, 4, 8).find("Unsupported dims") != std::string::npos);
    EXPECT(construct_msg(128, 512, 4, 8).find("Unsupported nlists") != std::string::npos);
    for (int nlist : {262144, 524288}) {
        std::string m = construct_msg(128, nlist, 3, 8);
        EXPECT(m.find("Unsupported nlists") == std::string::npos);
        EXPECT(m.find("Unsupported msubs") != std::string::npos);
    }
    EXPECT(construct_msg(128, 1024, 4, 4).find("Unsupported nbits") != std::string::npos);
    {
        // merge of two shards' results (FR/ascend/impl/AscendIndexImpl.cpp:587-640): invalid labels are
        // skipped, equal distances go to the lower shard, short results are padded
        std::vector<std::vector<float>> dist = {{1.f, 2.f, 5.f}, {2.f, 3.f, 4.f}};
        std::vector<std::vector<faiss::idx_t>> label = {{7, -1, 9}, {20, 21, -1}};
        float out_d[3];
        faiss::idx_t out_l[3];
        mergeSearchResult(dist, label, 1, 3, faiss::METRIC_L2, out_d, out_l);
        EXPECT(out_l[0] == 7 && out_l[1] == 20 && out_l[2] == 21);
        EXPECT(out_d[0] == 1.f && out_d[1] == 2.f && out_d[2] == 3.f);
    }
    if (argc > 1 && std::strcmp(argv[1], "gpu") == 0) {
        const int d = 128, nlist = 1024, M = 16, n = 40000, nq = 16, k = 5;
        std::mt19937 gen(1);
        std::normal_distribution<float> nd;
        std::vector<float> x((size_t)n * d);
        for (auto &v : x) {
            v = nd(gen);
        }
        AscendIndexIVFPQConfig conf({0});
        conf.niter = 3;
        AscendIndexIVFPQ index(d, faiss::METRIC_L2, nlist, M, 8, conf);
        EXPECT(!index.is_trained);
        index.train(n, x.data());
        index.add(n, x.data());
        EXPECT(index.ntotal == n);
        index.setNumProbes(32);
        std::vector<float> D((size_t)nq * k);
        std::vector<faiss::idx_t> I((size_t)nq * k);
        index.search(nq, x.data(), k, D.data(), I.data());
        int self = 0;
        for (int i = 0; i < nq; i++) {
            self += I[(size_t)i * k] == i;
        }
        EXPECT(self >= nq - 1);
        size_t total = 0;
        for (int l = 0; l < nlist; l++) {
            total += index.getListLength(l);
        }
        EXPECT(total == (size_t)n);
        // file form of copyTo / copyFrom: a second object loads what the first wrote
        const std::string path = std::string(argc > 2 ? argv[2] : "/tmp") + "/wrapper_test.faissindex";
        index.writeFaiss(path.c_str());
        AscendIndexIVFPQ other(d, faiss::METRIC_L2, nlist, M, 8, conf);
        other.readFaiss(path.c_str());
        EXPECT(other.is_trained && other.ntotal == n && other.getNumProbes() == 32);
        std::vector<float> D2((size_t)nq * k);
        std::vector<faiss::idx_t> I2((size_t)nq * k);
        other.search(nq, x.data(), k, D2.data(), I2.data());
        EXPECT(I2 == I && D2 == D);
        std::remove(path.c_str());
        AscendIndexIVFPQ wrong(d, faiss::METRIC_L2, 2048, M, 8, conf);
        bool threw = false;
        try {
            index.writeFaiss(path.c_str());
            wrong.readFaiss(path.c_str());
        } catch (const faiss::FaissException &) {
            threw = true;
        }
        EXPECT(threw);
        std::remove(path.c_str());
        AscendIndexFlatL2 flat(d);
        flat.add(n, x.data());
        flat.search(nq, x.data(), k, D.data(), I.data());
        for (int i = 0; i < nq; i++) {
            EXPECT(I[(size_t)i * k] == i);
        }
    }
    std::printf(failures ? "wrapper test FAILED\n" : "wrapper test ok\n");
    return failures ? 1 : 0;
}
