// Host-side check of the C++ wrappers: constructor validation messages as in
// FR/ut/TestAscendIndexUTIVFPQ.cpp:77-184.  With a GPU present (argv[1] == "gpu") it also runs a
// tiny train/add/search through the class interface.
#include <cfloat>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "ascend/AscendCloner.h"
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
        conf.strictReferenceParams = true;   // the reference's whitelists and messages
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
        conf.cp.niter = 3;                       // ClusteringParameters of the coarse quantizer (AscendIndexIVFConfig)
        conf.useKmeansPP = true;                 // accepted, changes nothing here
        AscendIndexIVFPQ index(d, faiss::METRIC_L2, nlist, M, 8, conf);
        EXPECT(!index.is_trained);
        index.train(n, x.data());
        // the levels of the hierarchy: AscendIndexIVFPQ -> AscendIndexIVF -> AscendIndex -> faiss::Index
        AscendIndexIVF *ivf = &index;
        AscendIndex *base = ivf;
        faiss::Index *root = base;
        base->reserveMemory((size_t)n);
        root->add(n, x.data());
        EXPECT(index.ntotal == n && ivf->getNumLists() == nlist && base->getDeviceList().size() == 1);
        EXPECT(base->reclaimMemory() > 0);
        ivf->setNumProbes(32);
        EXPECT(ivf->getNumProbes() == 32);
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
        {
            // remove_ids(const IDSelector &) on the second object, through the root of the hierarchy
            faiss::Index *other_root = &other;
            EXPECT(other_root->remove_ids(faiss::IDSelectorRange(10, 20)) == 10 && other.ntotal == n - 10);
            const faiss::idx_t some[] = {0, 5, 15, 5};      // 15 has left already
            EXPECT(other_root->remove_ids(faiss::IDSelectorBatch(4, some)) == 2 && other.ntotal == n - 12);
            struct EndsIn77 : faiss::IDSelector {
                bool is_member(faiss::idx_t id) const override { return id % 100 == 77; }
            };
            EXPECT(other_root->remove_ids(EndsIn77()) == (size_t)((n - 78) / 100 + 1));
            other.search(nq, x.data(), k, D2.data(), I2.data());
            bool none_left = true;
            for (size_t i = 0; i < I2.size(); i++) {
                const faiss::idx_t id = I2[i];
                none_left = none_left && !(id >= 10 && id < 20) && id != 0 && id != 5 && id % 100 != 77;
            }
            EXPECT(none_left && I2[0] >= 0);
        }
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
        {
            // copyTo / copyFrom through faiss::IndexIVFPQ (FR/ascend/impl/AscendIndexIVFPQImpl.cpp:392-508)
            faiss::IndexIVFPQ cpu;
            index.copyTo(&cpu);
            EXPECT(cpu.ntotal == n && cpu.nlist == (size_t)nlist && cpu.nprobe == 32 && !cpu.by_residual);
            EXPECT(cpu.pq.M == (size_t)M && cpu.pq.dsub == (size_t)(d / M) && cpu.quantizer->ntotal == nlist);
            size_t in_lists = 0;
            for (size_t l = 0; l < cpu.nlist; l++) {
                in_lists += cpu.invlists->list_size(l);
            }
            EXPECT(in_lists == (size_t)n);
            AscendIndexIVFPQConfig other_conf({0});
            AscendIndexIVFPQ from_cpu(d, faiss::METRIC_L2, 2048, 8, 8, other_conf);   // another shape: overwritten
            from_cpu.copyFrom(&cpu);
            EXPECT(from_cpu.is_trained && from_cpu.ntotal == n && from_cpu.getNumLists() == nlist &&
                   from_cpu.getNumProbes() == 32);
            std::vector<float> D3((size_t)nq * k);
            std::vector<faiss::idx_t> I3((size_t)nq * k);
            from_cpu.search(nq, x.data(), k, D3.data(), I3.data());
            EXPECT(I3 == I && D3 == D);
            std::vector<uint8_t> ca, cb2;
            std::vector<ascend_idx_t> ia, ib;
            index.getListCodesAndIds(5, ca, ia);
            from_cpu.getListCodesAndIds(5, cb2, ib);
            EXPECT(ca == cb2 && ia == ib);
            cpu.by_residual = true;   // codes of residuals can not be searched against raw queries: refused
            bool refused = false;
            try {
                from_cpu.copyFrom(&cpu);
            } catch (const faiss::FaissException &e) {
                refused = std::string(e.what()).find("by_residual") != std::string::npos;
            }
            EXPECT(refused && from_cpu.ntotal == n);
        }
        AscendIndexFlatL2 flat(d);
        AscendIndex *flat_base = &flat;
        EXPECT(flat_base->reclaimMemory() == 0);
        flat.add(n, x.data());
        flat.search(nq, x.data(), k, D.data(), I.data());
        for (int i = 0; i < nq; i++) {
            EXPECT(I[(size_t)i * k] == i);
        }
        faiss::IndexFlatL2 cpu_flat(d);
        flat.copyTo(&cpu_flat);
        EXPECT(cpu_flat.ntotal == n && std::memcmp(cpu_flat.get_xb(), x.data(), x.size() * sizeof(float)) == 0);
        AscendIndexFlat flat2(&cpu_flat);
        EXPECT(flat2.ntotal == n);
        // remove_ids through the faiss::Index interface: a range, a batch, and a selector of the caller's own
        {
            faiss::Index *as_index = &flat2;
            EXPECT(as_index->remove_ids(faiss::IDSelectorRange(n - 2, n + 5)) == 2 && flat2.ntotal == n - 2);
            const faiss::idx_t some[] = {0, 3, 3, n + 7};
            EXPECT(as_index->remove_ids(faiss::IDSelectorBatch(4, some)) == 2 && flat2.ntotal == n - 4);
            std::vector<faiss::idx_t> map;
            flat2.getIdxMap(0, map);
            // the holes 3 and 0, in that order, took the vectors that were last: n - 3, then n - 4
            EXPECT((faiss::idx_t)map.size() == n - 4 && map[3] == n - 3 && map[0] == n - 4 && map[1] == 1);
            struct Multiples : faiss::IDSelector {
                bool is_member(faiss::idx_t id) const override { return id % 100 == 1; }
            };
            const size_t expect = (size_t)((n - 3 - 1) / 100 + 1);   // 1, 101, ... among the ids up to n - 3 that are left
            EXPECT(as_index->remove_ids(Multiples()) == expect && flat2.ntotal == n - 4 - (faiss::idx_t)expect);
            flat2.search(1, x.data() + (size_t)5 * d, 1, D.data(), I.data());
            EXPECT(I[0] == 5);
        }
        // user ids in and out through faiss::IndexIDMap, and the calls with IEEE half inputs
        {
            faiss::IndexFlatL2 rows(d);
            faiss::IndexIDMap with_ids(&rows);
            std::vector<faiss::idx_t> user_ids(100);
            for (int i = 0; i < 100; i++) {
                user_ids[(size_t)i] = 7000 + 3 * i;
            }
            with_ids.add_with_ids(100, x.data(), user_ids.data());
            AscendIndexFlat from_map(&with_ids);
            EXPECT(from_map.ntotal == 100);
            from_map.search(1, x.data() + (size_t)9 * d, 1, D.data(), I.data());
            EXPECT(I[0] == 7027);
            faiss::IndexFlatL2 rows_back(d);
            faiss::IndexIDMap back(&rows_back);
            from_map.copyTo(&back);
            EXPECT(back.ntotal == 100 && back.id_map == user_ids &&
                   std::memcmp(rows_back.get_xb(), x.data(), (size_t)100 * d * sizeof(float)) == 0);
            // halves: 1.0, -2.0, 0.5, the smallest subnormal, 65504
            EXPECT(ixaHalfToFloat(0x3c00) == 1.0f && ixaHalfToFloat(0xc000) == -2.0f && ixaHalfToFloat(0x3800) == 0.5f &&
                   ixaHalfToFloat(0x0001) == 5.9604644775390625e-08f && ixaHalfToFloat(0x7bff) == 65504.0f);
            std::vector<uint16_t> halves((size_t)3 * d, 0x3c00);     // three rows of ones ...
            halves[(size_t)d] = 0xc000;                              // ... the second starts with -2
            halves[(size_t)2 * d + 1] = 0x3800;                      // ... the third has a 0.5
            AscendIndexFlat half_index(d, faiss::METRIC_L2);
            AscendIndex *half_base = &half_index;
            half_base->add(3, halves.data());
            EXPECT(half_index.ntotal == 3);
            half_base->search(1, halves.data() + (size_t)d, 2, D.data(), I.data());
            EXPECT(I[0] == 1 && D[0] == 0.f && I[1] == 0 && D[1] == 9.f);
        }
        // the cloner: device -> CPU -> device, Flat (ids travel in an IndexIDMap) and IVFPQ
        {
            std::unique_ptr<faiss::Index> cpu_copy(index_ascend_to_cpu(&flat));
            auto *as_map = dynamic_cast<faiss::IndexIDMap *>(cpu_copy.get());
            EXPECT(as_map != nullptr && as_map->ntotal == n && as_map->own_fields && (faiss::idx_t)as_map->id_map.size() == n &&
                   as_map->id_map[7] == 7);
            std::unique_ptr<faiss::Index> device_copy(index_cpu_to_ascend({0}, cpu_copy.get()));
            EXPECT(dynamic_cast<AscendIndexFlat *>(device_copy.get()) != nullptr && device_copy->ntotal == n);
            device_copy->search(nq, x.data(), k, D.data(), I.data());
            for (int i = 0; i < nq; i++) {
                EXPECT(I[(size_t)i * k] == i);
            }
            std::unique_ptr<faiss::Index> pq_cpu(index_ascend_to_cpu(&index));
            EXPECT(dynamic_cast<faiss::IndexIVFPQ *>(pq_cpu.get()) != nullptr && pq_cpu->ntotal == n);
            AscendClonerOptions options;
            options.reserveVecs = 1000;
            std::unique_ptr<faiss::Index> pq_device(index_cpu_to_ascend(std::vector<int>{0}, pq_cpu.get(), &options));
            auto *pq_again = dynamic_cast<AscendIndexIVFPQ *>(pq_device.get());
            EXPECT(pq_again != nullptr && pq_again->ntotal == n && pq_again->getNumProbes() == 32);
            std::vector<float> Dc((size_t)nq * k);
            std::vector<faiss::idx_t> Ic((size_t)nq * k);
            index.search(nq, x.data(), k, D.data(), I.data());
            pq_again->search(nq, x.data(), k, Dc.data(), Ic.data());
            EXPECT(Ic == I && Dc == D);
            bool refused = false;
            try {
                AscendIndexInt8Flat not_cloneable(64);
                faiss::IndexFlatL2 other_kind(8);
                faiss::IndexIDMap map_over_map(&other_kind);
                faiss::IndexIDMap outer(&map_over_map);
                index_cpu_to_ascend({0}, &outer);
            } catch (const faiss::FaissException &e) {
                refused = std::string(e.what()).find("not supported") != std::string::npos;
            }
            EXPECT(refused);
        }
        // int8: AscendIndexInt8Flat -> AscendIndexInt8
        std::vector<int8_t> b((size_t)4096 * 64);
        for (auto &v : b) {
            v = (int8_t)((int)(gen() % 255) - 127);
        }
        AscendIndexInt8Flat i8(64);
        AscendIndexInt8 *i8_base = &i8;
        i8_base->add(4096, b.data());
        std::vector<float> Di((size_t)4 * 3);
        std::vector<faiss::idx_t> Ii((size_t)4 * 3);
        i8_base->search(4, b.data(), 3, Di.data(), Ii.data());
        for (int i = 0; i < 4; i++) {
            EXPECT(Ii[(size_t)i * 3] == i && Di[(size_t)i * 3] == 0.f);
        }
        {
            // masks: the query that is base vector 0 may only see vectors 8..15 -> its nearest comes from there
            std::vector<uint8_t> mask((size_t)4096 / 8, 0);
            mask[1] = 0xff;
            i8.search_with_masks(1, b.data(), 3, Di.data(), Ii.data(), mask.data());
            EXPECT(Ii[0] >= 8 && Ii[0] < 16 && Ii[1] >= 8 && Ii[1] < 16 && Di[0] > 0.f && Di[0] <= Di[1]);
            mask[0] = 0x01;
            i8.search_with_masks(1, b.data(), 3, Di.data(), Ii.data(), mask.data());
            EXPECT(Ii[0] == 0 && Di[0] == 0.f);
            std::vector<uint8_t> fmask((size_t)(n + 7) / 8, 0);
            fmask[0] = 0x04;                                  // only vector 2
            flat.search_with_masks(1, x.data(), 2, D.data(), I.data(), fmask.data());
            EXPECT(I[0] == 2 && I[1] == -1 && D[1] == FLT_MAX);
        }
        {
            // int8 cloner: device -> IndexIDMap over IndexScalarQuantizer -> device
            std::unique_ptr<faiss::Index> cpu8(index_int8_ascend_to_cpu(i8_base));
            auto *map8c = dynamic_cast<faiss::IndexIDMap *>(cpu8.get());
            auto *sq8 = map8c ? dynamic_cast<faiss::IndexScalarQuantizer *>(map8c->index) : nullptr;
            EXPECT(sq8 != nullptr && map8c->ntotal == 4096 && sq8->codes.size() == b.size() &&
                   std::memcmp(sq8->codes.data(), b.data(), b.size()) == 0 && map8c->id_map[4095] == 4095);
            for (auto &id : map8c->id_map) {
                id += 100000;
            }
            std::unique_ptr<AscendIndexInt8> back8(index_int8_cpu_to_ascend({0}, cpu8.get()));
            EXPECT(back8->getNTotal() == 4096 && back8->getDim() == 64);
            back8->search(2, b.data() + (size_t)17 * 64, 1, Di.data(), Ii.data());
            EXPECT(Ii[0] == 100017 && Ii[1] == 100018 && Di[0] == 0.f);
            AscendIndexInt8Flat from_codes(sq8);          // without ids: numbered from 0
            from_codes.search(1, b.data() + (size_t)5 * 64, 1, Di.data(), Ii.data());
            EXPECT(from_codes.getNTotal() == 4096 && Ii[0] == 5);
        }
        std::vector<faiss::idx_t> nearest(4);
        i8_base->assign(4, b.data(), nearest.data());
        EXPECT(nearest[0] == 0 && nearest[3] == 3);
        i8.setPageSize(8);
        EXPECT(i8_base->remove_ids(faiss::IDSelectorRange(1, 3)) == 2 && i8_base->getNTotal() == 4094);
        std::vector<faiss::idx_t> map8;
        i8.getIdxMap(0, map8);
        EXPECT(map8.size() == 4094 && map8[0] == 0 && map8[2] == 4095 && map8[1] == 4094);
        i8_base->search(1, b.data() + (size_t)4095 * 64, 3, Di.data(), Ii.data());
        EXPECT(Ii[0] == 4095 && Di[0] == 0.f);
    }
    std::printf(failures ? "wrapper test FAILED\n" : "wrapper test ok\n");
    return failures ? 1 : 0;
}
