// Stages 2-4 of IVFPQ search fused into one kernel: per-query PQ lookup table built straight into
// LDS, ADC scan of the probed inverted lists, wavefront-level top-k, workgroup merge.
//
// Replaces, for one GPU, the reference's L2 and L3 levels
// (FR/ascenddaemon/impl/IndexIVFPQ.cpp:2151, 2166-2349):
//   op AscendcIvfpqSubspaceDistance  (FR/ops/ascendc/op_kernel/ascendc_ivfpq_subspace_distance.cpp:419-463)
//   op AscendcIvfpqSearchDistanceL2  (FR/ops/ascendc/op_kernel/ascendc_ivfpq_search_distance_topk.h:39-93, 556-810)
//   op TopkIvfpqL3                   (FR/ops/cpukernel/impl/topk_ivfpq_l3_cpu_kernel.cpp:176-250)
// The reference round-trips the LUT and a [B,128,262144] distance scratch through global memory and
// selects a fixed top-320; here the LUT never leaves LDS, no distance is ever written to HBM and
// the selection is exactly top-k.
//
// Layout of one inverted list in the code arena: list l owns slots [list_off[l], list_off[l] +
// roundup64(list_len[l])); slot s holds M code bytes at codes + s*M and its id at ids[s].
// Code layout 0 ("row"): byte j of a slot is sub-quantizer j.
// Code layout 1 ("rot32", M % 32 == 0): byte j of the slot at list position p holds sub-quantizer
//   32*(j/32) + ((j + p) % 32).  With the LUT stored k-major (word k*M + m) the 32 lanes of a half
//   wavefront then read 32 different sub-quantizers, i.e. 32 different LDS banks, at every step,
//   whatever their code values are.
#include "scan.h"

#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "topk.h"

namespace ixa {

template <typename T>
__device__ __forceinline__ T to_lut(float v);
template <>
__device__ __forceinline__ float to_lut<float>(float v)
{
    return v;
}
template <>
__device__ __forceinline__ __half to_lut<__half>(float v)
{
    return __float2half_rn(v);
}
__device__ __forceinline__ float from_lut(float v) { return v; }
__device__ __forceinline__ float from_lut(__half v) { return __half2float(v); }

// Half-precision LUT under the rot32 code layout.  Two halves share one 32-bit LDS word, so "32
// lanes read 32 different sub-quantizers" only means 32 different banks if the words they read are
// 32 different words modulo the 32 banks, whatever the code values.  Sub-quantizer r of a 32-block
// sits at byte R(r) = 4 r + 2 (r >> 4) of its codeword's row: word r, low half for r < 16, high half
// above.
//   * Blocks are paired.  Block pair p owns 32 KB, codeword kk a row of 128 bytes in it; the even
//     block starts at byte 0 of the row, the odd block at byte 64, so that its sub-quantizers 16..31
//     land in words 0..15 of the NEXT row -- in the half that row's even block (r < 16) leaves free.
//     A lane's bank is r (even block) or r + 16 mod 32 (odd block): no conflicts.
//   * A last block without partner has rows of 64 bytes, so that its sub-quantizers 16..31 reach into
//     the next row in the same way.  Lanes r and r ^ 16 then share a bank whenever their codes differ
//     in parity (a two-way conflict on most reads of that block), which costs less than the two extra
//     address instructions per lookup of the conflict-free alternative, pairing codewords (row kk / 2,
//     half kk % 2): the scan is bound by vector instructions.
// Every address is (code << 7 or 6) + a per-lane constant + an immediate: one shift-add.  The last
// row's upper half needs 64 bytes beyond M * 512.
// (Giving the unpaired block 32 KB of its own with fp32 words has neither cost, but the larger LUT
// costs a resident workgroup at M = 96: measured slower.)
__host__ __device__ __forceinline__ int rot32_half_slot(int nblocks, int m, int kk)
{
    const int b = m >> 5, r = m & 31;
    const int in_row = r * 4 + 2 * (r >> 4);
    int byte;
    if (b < (nblocks & ~1)) {
        byte = (b >> 1) * 32768 + kk * 128 + 64 * (b & 1) + in_row;
    } else {
        byte = (nblocks >> 1) * 32768 + kk * 64 + in_row;
    }
    return byte >> 1;
}

// One 64-code group of a probed list, as a wavefront sees it.
struct GroupRef {
    uint32_t slot;  // arena slot of this lane's code
    bool valid;     // lane is inside the list
};

// MT > 0: compile-time number of sub-quantizers; MT == 0: run-time p.M with byte loads.
// W: wavefronts per workgroup (the workgroup serves one query, or one split of a query).
// SHARED: one workgroup-wide candidate pool (BlockPool) instead of W private ones (WavePool); the
// choice for k so large that private pools would leave room for only a few waves per CU.
// The half-LUT rot32 variants are held to 128 registers (4 waves per SIMD): their LDS plan admits
// two 8-wave workgroups per CU and the register allocator would otherwise trade that away.
// Byte j of a 32-bit word times 2^SH as one instruction: a left shift whose shifted operand is selected by
// byte (sub-dword addressing), so no separate extraction is needed.
template <int SH>
__device__ __forceinline__ uint32_t byte_times_pow2(uint32_t w, int j)
{
    uint32_t r;
    const uint32_t sh = SH;
    switch (j) {
        case 0:
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
                : "=v"(r) : "s"(sh), "v"(w));
            break;
        case 1:
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1"
                : "=v"(r) : "s"(sh), "v"(w));
            break;
        case 2:
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2"
                : "=v"(r) : "s"(sh), "v"(w));
            break;
        default:
            asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3"
                : "=v"(r) : "s"(sh), "v"(w));
            break;
    }
    return r;
}

template <int MT, typename LutT, int LAYOUT, int W, bool SHARED>
__global__ __launch_bounds__(W * 64, (LAYOUT == 1 && sizeof(LutT) == 2 && !SHARED) ? 4 : 1) void ivfpq_scan_kernel(
    ScanParams p)
{
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int NT = W * 64;
    const int M = MT > 0 ? MT : p.M;
    LutT *lut = reinterpret_cast<LutT *>(smem_raw);
    float *qs = reinterpret_cast<float *>(smem_raw + p.off_query);
    key_t *pools = reinterpret_cast<key_t *>(smem_raw + p.off_pools);
    float *share = reinterpret_cast<float *>(smem_raw + p.off_misc);    // W: score at rank ceil(k/W) per wave
    int *counts = reinterpret_cast<int *>(share + W);                   // W
    uint32_t *t_off = reinterpret_cast<uint32_t *>(smem_raw + p.off_table);  // first slot of local list i
    int *t_len = reinterpret_cast<int *>(t_off + p.table_n);                  // its length
    int *t_gend = t_len + p.table_n;                                          // groups up to and incl. list i

    const int tid = threadIdx.x, lane = tid & 63;
    // the wavefront index is uniform: keeping it (and everything derived from it) in scalar
    // registers turns the group bookkeeping below into scalar code
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups are dealt to the 8 XCDs round-robin.  With xcd_chunks the query order is cut into 8
    // contiguous chunks, one per XCD, so that neighbouring queries (which tend to probe the same
    // lists when the caller orders them by locality) share one L2.
    int64_t qslot = blockIdx.x / p.nsplit;
    if (p.xcd_chunks) {
        const int64_t per = (p.nq + 7) / 8;
        qslot = (qslot & 7) * per + (qslot >> 3);
        if (qslot >= p.nq) {
            return;
        }
    }
    const int64_t q = p.order ? p.order[qslot] : qslot;
    const int split = blockIdx.x % p.nsplit;

    // ---- list table of this workgroup: local list i = probe rank split + i * nsplit
    const int nlocal = (p.nprobe - split + p.nsplit - 1) / p.nsplit;
    for (int j = tid; j < p.d; j += NT) {
        qs[j] = p.queries[q * p.d + j];
    }
    if (tid < W) {
        share[tid] = __builtin_inff();
    }
    for (int i = tid; i < nlocal; i += NT) {
        const int l = p.probes[q * p.nprobe + split + i * p.nsplit];
        const bool has = (uint32_t)l < (uint32_t)p.nlist;   // anything else is "no list", whatever the caller left there
        const int len = has ? p.list_len[l] : 0;
        t_len[i] = len;
        t_off[i] = has ? (uint32_t)p.list_off[l] : 0u;
    }
    __syncthreads();
    if (wave == 0) {
        // inclusive prefix sum of the group counts, 64 lists at a time
        int carry = 0;
        for (int base = 0; base < nlocal; base += 64) {
            const int i = base + lane;
            int g = i < nlocal ? (t_len[i] + 63) >> 6 : 0;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                int up = __shfl_up(g, o);
                if (lane >= o) {
                    g += up;
                }
            }
            if (i < nlocal) {
                t_gend[i] = carry + g;
            }
            carry += __shfl(g, 63);
        }
    }

    // ---- stage 2: LUT into LDS.  Thread t owns codeword k = t % 256 of every (NT/256)-th sub-quantizer.
    // For the usual sub-vector lengths the codewords of four entries are loaded before the first is
    // used: one memory round trip per four entries instead of one per entry, which is most of a
    // workgroup's start-up time (and of a small batch's latency).  The arithmetic is the same either way.
    {
        const int kk = tid & 255;
        auto store_entry = [&](int m, float ip, float qn, float cbn) {
            float v;
            if (p.metric == kMetricL2) {
                v = __fadd_rn(__fadd_rn(cbn, qn), __fmul_rn(ip, -2.0f));
            } else {
                v = -ip;  // minimise the negated inner product
            }
            if constexpr (LAYOUT == 2) {
                // xor48: rows of 64 words per codeword; sub-quantizers 32..47 are stored twice
                lut[kk * 64 + m] = to_lut<LutT>(v);
                if (m >= 32) {
                    lut[kk * 64 + m + 16] = to_lut<LutT>(v);
                }
            } else {
                int slot = LAYOUT == 1 ? kk * M + m : m * 256 + kk;
                if constexpr (LAYOUT == 1 && sizeof(LutT) == 2) {
                    slot = rot32_half_slot(M / 32, m, kk);
                }
                lut[slot] = to_lut<LutT>(v);
            }
        };
        const bool l2 = p.metric == kMetricL2;
        auto build = [&](auto dsc) {
            constexpr int DS = decltype(dsc)::value;
            constexpr int kAhead = 4, kStep = NT / 256;
            for (int m0 = tid >> 8; m0 < M; m0 += kAhead * kStep) {
                float cwv[kAhead][DS], cbn[kAhead];
#pragma unroll
                for (int u = 0; u < kAhead; u++) {
                    const int m = m0 + u * kStep;
                    cbn[u] = 0.f;
                    if (m < M) {
                        const float *cw = p.codebook + ((int64_t)m * 256 + kk) * DS;
                        if constexpr (DS % 4 == 0) {
#pragma unroll
                            for (int t = 0; t < DS; t += 4) {
                                const float4 x = *reinterpret_cast<const float4 *>(cw + t);
                                cwv[u][t] = x.x;
                                cwv[u][t + 1] = x.y;
                                cwv[u][t + 2] = x.z;
                                cwv[u][t + 3] = x.w;
                            }
                        } else if constexpr (DS == 2) {
                            const float2 x = *reinterpret_cast<const float2 *>(cw);
                            cwv[u][0] = x.x;
                            cwv[u][1] = x.y;
                        } else {
#pragma unroll
                            for (int t = 0; t < DS; t++) {
                                cwv[u][t] = cw[t];
                            }
                        }
                        if (l2) {
                            cbn[u] = p.cb_norms[m * 256 + kk];
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < kAhead; u++) {
                    const int m = m0 + u * kStep;
                    if (m < M) {
                        const float *qm = qs + m * DS;
                        float ip = 0.f, qn = 0.f;
#pragma unroll
                        for (int t = 0; t < DS; t++) {
                            const float qv = qm[t];
                            ip = __fadd_rn(ip, __fmul_rn(qv, cwv[u][t]));
                            qn = __fadd_rn(qn, __fmul_rn(qv, qv));
                        }
                        store_entry(m, ip, qn, cbn[u]);
                    }
                }
            }
        };
        const int dsub = p.dsub;
        if (dsub == 4) {
            build(std::integral_constant<int, 4>{});
        } else if (dsub == 8) {
            build(std::integral_constant<int, 8>{});
        } else if (dsub == 2) {
            build(std::integral_constant<int, 2>{});
        } else if (dsub == 1) {
            build(std::integral_constant<int, 1>{});
        } else if (dsub % 16 == 0) {
            // long sub-vectors (128 dimensions in 2, 4 or 8 sub-quantizers): sixteen codeword floats per memory
            // round trip instead of one, accumulated in the same order
            for (int m = tid >> 8; m < M; m += NT / 256) {
                const float *qm = qs + m * dsub;
                const float4 *cw = reinterpret_cast<const float4 *>(p.codebook + ((int64_t)m * 256 + kk) * dsub);
                float ip = 0.f, qn = 0.f;
                for (int t0 = 0; t0 < dsub; t0 += 16) {
                    float4 c[4];
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        c[u] = cw[(t0 >> 2) + u];
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const float cv[4] = {c[u].x, c[u].y, c[u].z, c[u].w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float qv = qm[t0 + 4 * u + j];
                            ip = __fadd_rn(ip, __fmul_rn(qv, cv[j]));
                            qn = __fadd_rn(qn, __fmul_rn(qv, qv));
                        }
                    }
                }
                store_entry(m, ip, qn, l2 ? p.cb_norms[m * 256 + kk] : 0.f);
            }
        } else {
            for (int m = tid >> 8; m < M; m += NT / 256) {
                const float *qm = qs + m * dsub;
                const float *cw = p.codebook + ((int64_t)m * 256 + kk) * dsub;
                float ip = 0.f, qn = 0.f;
                for (int t = 0; t < dsub; t++) {
                    float qv = qm[t];
                    ip = __fadd_rn(ip, __fmul_rn(qv, cw[t]));
                    qn = __fadd_rn(qn, __fmul_rn(qv, qv));
                }
                store_entry(m, ip, qn, l2 ? p.cb_norms[m * 256 + kk] : 0.f);
            }
        }
    }
    __syncthreads();

    // ---- stages 3 + 4: the probed lists form one sequence of 64-code groups; wavefront w takes
    // groups w, w + W, ... of that sequence, so the waves stay balanced whatever the list lengths.
    WavePool<float> pool;
    BlockPool<W> bpool;
    if constexpr (SHARED) {
        bpool.init(pools, p.cap, p.k, reinterpret_cast<int *>(smem_raw + p.off_hist),
                   reinterpret_cast<BlockPoolCtl *>(counts + W), tid);
        __syncthreads();
    } else {
        pool.init(pools + wave * p.cap, p.cap, p.k);
    }
    const int l32 = lane & 31;
    const int total = nlocal > 0 ? __builtin_amdgcn_readfirstlane(t_gend[nlocal - 1]) : 0;
    int li = 0;          // list the current group belongs to (monotone, wave-uniform)
    int gstart = 0;      // first group of that list
    int gend = nlocal > 0 ? __builtin_amdgcn_readfirstlane(t_gend[0]) : 0;

    auto locate = [&](int G) -> GroupRef {
        while (G >= gend) {
            gstart = gend;
            li++;
            gend = __builtin_amdgcn_readfirstlane(t_gend[li]);
        }
        const int pos = ((G - gstart) << 6) + lane;
        GroupRef r;
        r.slot = (uint32_t)__builtin_amdgcn_readfirstlane((int)t_off[li]) + (uint32_t)pos;
        r.valid = pos < __builtin_amdgcn_readfirstlane(t_len[li]);
        return r;
    };

    constexpr int NW = MT > 0 ? (MT + 3) / 4 : 1;
    // Lanes past the end of a list load nothing when a code is long: with 96-byte codes the padding of the last
    // group is 5 % of the bytes of a 600-code list, and the launch is bound by the bytes it fetches (20M x 96 B,
    // 4096 queries x 128 lists: 5.2 -> 4.95 ms).  With short codes the exec-mask bookkeeping costs more than the bytes
    // (10M x 32 B, 10000 queries x 64 lists: 1.59 -> 1.61 ms), so those kernels load whole groups.
    constexpr bool kSkipPadding = MT >= 64;
    auto load_codes = [&](uint32_t slot, uint32_t (&w)[NW]) {
        if (MT == 0) {
            return;
        }
        const uint8_t *cp = p.codes + (int64_t)slot * MT;
        if (MT % 16 == 0) {
#pragma unroll
            for (int v = 0; v < MT / 16; v++) {
                uint4 u = reinterpret_cast<const uint4 *>(cp)[v];
                w[(4 * v + 0) % NW] = u.x;
                w[(4 * v + 1) % NW] = u.y;
                w[(4 * v + 2) % NW] = u.z;
                w[(4 * v + 3) % NW] = u.w;
            }
        } else if (MT % 8 == 0) {
#pragma unroll
            for (int v = 0; v < MT / 8; v++) {
                uint2 u = reinterpret_cast<const uint2 *>(cp)[v];
                w[(2 * v + 0) % NW] = u.x;
                w[(2 * v + 1) % NW] = u.y;
            }
        } else if (MT % 4 == 0) {
#pragma unroll
            for (int v = 0; v < MT / 4; v++) {
                w[v % NW] = reinterpret_cast<const uint32_t *>(cp)[v];
            }
        } else if (MT == 2) {
            w[0] = *reinterpret_cast<const uint16_t *>(cp);   // slots are 2 bytes apart: always aligned
        } else {
#pragma unroll
            for (int v = 0; v < NW; v++) {
                w[v] = 0;
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                w[(m >> 2) % NW] |= (uint32_t)cp[m] << (8 * (m & 3));
            }
        }
    };

    // LDS address of this lane's word in the first 32-word LUT row at each of the 32 rotation steps;
    // kept in registers (opaque to the optimiser, which would otherwise recompute them per lookup),
    // so that a lookup's address is one shift-add of the code
    typedef __attribute__((address_space(3))) const uint16_t lds_half_t;
    uint32_t rot4[32];
    if constexpr (LAYOUT == 1 && sizeof(LutT) == 2) {
        const uint32_t lut_base =
            (uint32_t) reinterpret_cast<size_t>((__attribute__((address_space(3))) const unsigned char *)lut);
#pragma unroll
        for (int j = 0; j < 32; j++) {
            const uint32_t r = (uint32_t)((j + l32) & 31);
            rot4[j] = lut_base + (r << 2) + ((r >> 4) << 1);   // byte R(r) of a row (rot32_half_slot)
            asm volatile("" : "+v"(rot4[j]));
        }
    }
    auto adc = [&](uint32_t slot, const uint32_t (&w)[NW]) -> float {
        if (MT == 0) {
            const uint8_t *cp = p.codes + (int64_t)slot * M;
            float s = 0.f;
            for (int m = 0; m < M; m++) {
                s = __fadd_rn(s, from_lut(lut[m * 256 + cp[m]]));
            }
            return s;
        }
        if constexpr (LAYOUT == 1 && sizeof(LutT) == 2) {
            // half LUT in paired blocks or 64-byte rows (rot32_half_slot); the conversion to fp32 and the
            // addition are one v_fma_mix_f32 (half * 1.0 + fp32 accumulator: the same value as convert-then-add)
            constexpr int NB = MT / 32;
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const uint32_t ww = w[(m >> 2) % NW];
                const int b = m >> 5;
                const uint32_t r4 = rot4[m & 31];
                uint32_t off;
                uint32_t code = (ww >> (8 * (m & 3))) & 0xffu;
                asm("" : "+v"(code));   // keep extract-then-shift-add (two instructions for every byte)
                if (b < (NB & ~1)) {
                    off = ((code << 7) + r4) + (uint32_t)((b >> 1) * 32768 + 64 * (b & 1));
                } else {
                    off = ((code << 6) + r4) + (uint32_t)((NB >> 1) * 32768);
                }
                const uint32_t raw = *(lds_half_t *)(size_t)off;
                asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel_hi:[1,0,0]" : "+v"(acc[m & 3]) : "v"(raw));
            }
            return (acc[0] + acc[1]) + (acc[2] + acc[3]);
        } else if constexpr (LAYOUT == 2) {
            // xor48: byte address = (code << 8) + ((4 * l32) ^ (4 * c)) + block offset, c the step's
            // constant: one byte permute (code into bits 8..15), one xor-add, one fp add per lookup
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            const unsigned char *lb = reinterpret_cast<const unsigned char *>(lut);
            const uint32_t x4 = (uint32_t)l32 << 2;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const uint32_t ww = w[(m >> 2) % NW];
                const uint32_t code8 = __builtin_amdgcn_perm(0u, ww, 0x0c0c000cu | ((uint32_t)(m & 3) << 8));
                const uint32_t c4 = (uint32_t)(m < 32 ? m : (m & 15)) << 2;
                const uint32_t off = (x4 ^ c4) + code8 + (m < 32 ? 0u : 128u);
                acc[m & 3] += *reinterpret_cast<const float *>(lb + off);
            }
            return (acc[0] + acc[1]) + (acc[2] + acc[3]);
        } else if (LAYOUT == 1) {
            // any association is within tolerance: four independent partial sums
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int m = 0; m < MT; m++) {
                uint32_t code = (w[(m >> 2) % NW] >> (8 * (m & 3))) & 0xffu;
                asm("" : "+v"(code));   // keep extract-then-shift-add (two instructions for every byte)
                const int mm = (m & ~31) | ((m + l32) & 31);
                acc[m & 3] += from_lut(lut[code * MT + mm]);
            }
            return (acc[0] + acc[1]) + (acc[2] + acc[3]);
        }
        // row layout: m = 0..M-1 in sequence, the accumulation order of the reference's scalar path.  The byte
        // offset of the entry inside its 256-entry row is ONE instruction (a shift whose operand is byte m % 4 of
        // the code word) and the row's start is the load's immediate offset: two VALU instructions per lookup
        // with the addition, where extract, scale and add are three -- the scan loop is bound by VALU issue.
        // The LUT is the first thing in the workgroup's LDS and the kernel has no static LDS (the host checks
        // that before the first launch), so its LDS address is 0 and needs no addition either.
        typedef __attribute__((address_space(3))) const float lds_f32_t;
        float s = 0.f;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const uint32_t off = byte_times_pow2<sizeof(LutT) == 4 ? 2 : 1>(w[(m >> 2) % NW], m & 3);
            const uint32_t addr = (uint32_t)(m * 256 * sizeof(LutT)) + off;
            float v;
            if constexpr (sizeof(LutT) == 4) {
                v = *(lds_f32_t *)(size_t)addr;
            } else {
                v = __half2float(__ushort_as_half(*(lds_half_t *)(size_t)addr));
            }
            s = __fadd_rn(s, v);
        }
        return s;
    };

    // The largest of the W published rank-ceil(k/W) scores has >= k candidates at or below it
    // across the workgroup: a valid bound for every wave.
    const int share_rank = (p.k + W - 1) / W;
    auto adopt_shared = [&]() {
        float b = share[0];
#pragma unroll
        for (int i = 1; i < W; i++) {
            b = fmaxf(b, share[i]);
        }
        b = wave_uniform(b);
        pool.bound = b < pool.bound ? b : pool.bound;
    };
    // One step: start the loads of the group after next, evaluate the current group, offer it to
    // the pool.  Two register sets (a, b) alternate so that no code registers are ever copied; the
    // step is a macro so that both sets stay in registers (no address of either is ever taken).
    // PF: the step starts the next group's loads.  The loops below start them unconditionally (PF a literal) and
    // leave the last groups to a tail without them: behind a load that is issued under a condition the compiler
    // waits for EVERY outstanding load before it evaluates the current group, the one just requested included,
    // and a wavefront then walks its groups at one memory round trip each.
#define IXA_SCAN_STEP(G, CUR, WCUR, NXT, WNXT, PF)                                                    \
    do {                                                                                              \
        if (PF) {                                                                                     \
            NXT = locate((G) + W);                                                                    \
            if (!kSkipPadding || NXT.valid) { /* lanes past the list's end fetch nothing */           \
                load_codes(NXT.slot, WNXT); /* in flight while the current group is evaluated */      \
            }                                                                                         \
        }                                                                                             \
        const float s_ = adc(CUR.slot, WCUR);                                                         \
        const bool compacted_ =                                                                       \
            pool.push(CUR.valid && s_ <= pool.bound, s_, CUR.slot, lane, &share[wave], share_rank);   \
        if (compacted_ || ((G) & (16 * W - 1)) < W) {                                                 \
            adopt_shared();                                                                           \
        }                                                                                             \
    } while (0)
    // The same step for the shared pool: poll for a pending prune, evaluate, reserve-and-append;
    // a failed reservation is retried after the workgroup has pruned the pool.
#define IXA_SCAN_STEP_SHARED(G, CUR, WCUR, NXT, WNXT, PF)                                             \
    do {                                                                                              \
        if (PF) {                                                                                     \
            NXT = locate((G) + W);                                                                    \
            if (!kSkipPadding || NXT.valid) {                                                         \
                load_codes(NXT.slot, WNXT);                                                           \
            }                                                                                         \
        }                                                                                             \
        if (bpool.poll()) {                                                                           \
            bpool.rendezvous(tid);                                                                    \
        }                                                                                             \
        const float s_ = adc(CUR.slot, WCUR);                                                         \
        while (!bpool.try_push(CUR.valid && s_ <= bpool.bound, s_, CUR.slot, lane)) {                 \
            bpool.rendezvous(tid);                                                                    \
        }                                                                                             \
    } while (0)
    int total_keys;
    if constexpr (SHARED) {
        if (wave < total) {
            uint32_t wa[NW] = {}, wb[NW] = {};
            GroupRef ga = locate(wave), gb = ga;
            if (!kSkipPadding || ga.valid) {
                load_codes(ga.slot, wa);
            }
            if constexpr (W == 16) {
                // sixteen wavefronts hide the latency by themselves, and the plain loop measured 2.5 % faster
                // there (100M x 96, nprobe 256, k 1024: scan 4.34 against 4.44 ms)
                for (int G = wave; G < total; G += 2 * W) {
                    IXA_SCAN_STEP_SHARED(G, ga, wa, gb, wb, G + W < total);
                    if (G + W < total) {
                        IXA_SCAN_STEP_SHARED(G + W, gb, wb, ga, wa, G + 2 * W < total);
                    }
                }
            } else {
                int G = wave;
                for (; G + 2 * W < total; G += 2 * W) {   // the groups G, G + W and G + 2 W exist
                    IXA_SCAN_STEP_SHARED(G, ga, wa, gb, wb, 1);
                    IXA_SCAN_STEP_SHARED(G + W, gb, wb, ga, wa, 1);
                }
                if (G + W < total) {   // two groups left (the first is in set a), or one
                    IXA_SCAN_STEP_SHARED(G, ga, wa, gb, wb, 1);
                    IXA_SCAN_STEP_SHARED(G + W, gb, wb, ga, wa, 0);
                } else {
                    IXA_SCAN_STEP_SHARED(G, ga, wa, gb, wb, 0);
                }
            }
        }
        bpool.finish_wave(lane);
        while (!bpool.rendezvous(tid)) {
        }
        total_keys = bpool.sort_all(tid);
    } else {
        if (wave < total) {
            uint32_t wa[NW] = {}, wb[NW] = {};
            GroupRef ga = locate(wave), gb = ga;
            if (!kSkipPadding || ga.valid) {
                load_codes(ga.slot, wa);
            }
            int G = wave;
            for (; G + 2 * W < total; G += 2 * W) {   // the groups G, G + W and G + 2 W exist
                IXA_SCAN_STEP(G, ga, wa, gb, wb, 1);
                IXA_SCAN_STEP(G + W, gb, wb, ga, wa, 1);
            }
            if (G + W < total) {   // two groups left (the first is in set a), or one
                IXA_SCAN_STEP(G, ga, wa, gb, wb, 1);
                IXA_SCAN_STEP(G + W, gb, wb, ga, wa, 0);
            } else {
                IXA_SCAN_STEP(G, ga, wa, gb, wb, 0);
            }
        }
        __syncthreads();  // every wave has published its last value; the LUT is no longer needed
        adopt_shared();
        pool.finish(lane);
        if (lane == 0) {
            counts[wave] = pool.count;
        }
        total_keys = block_merge_pools<W>(pools, p.cap, counts, nullptr, 0, tid);
    }
#undef IXA_SCAN_STEP
#undef IXA_SCAN_STEP_SHARED
    const key_t *merge = pools;

    if (p.nsplit > 1) {
        key_t *dst = p.partial + ((int64_t)q * p.nsplit + split) * p.k;
        for (int i = tid; i < p.k; i += NT) {
            dst[i] = i < total_keys ? merge[i] : kEmptyKey;
        }
        return;
    }
    for (int i = tid; i < p.k; i += NT) {
        const key_t kk = i < total_keys ? merge[i] : kEmptyKey;
        const bool ok = kk != kEmptyKey;
        const float v = key_score(kk);
        const float pad = p.metric == kMetricL2 ? 3.402823466e+38f : -3.402823466e+38f;
        p.out_dist[q * p.k + i] = ok ? (p.metric == kMetricL2 ? v : -v) : pad;
        p.out_labels[q * p.k + i] = ok ? p.ids[key_index(kk)] : -1;
    }
}

// Merges the nsplit sorted partial lists of a query (tile merge, the role of op TopkIvfpqL3).
//
// 1. A bound from the slices' own order.  Every slice is sorted, so two of its keys bound the k-th smallest key
//    of the query from above: the last key of a slice that is full (that slice alone has k keys at or below it),
//    and the largest of the slices' keys at rank r = ceil(k / nsplit) (r keys of every slice lie at or below
//    it).  ONE pass over the nsplit x k keys (global memory / L2) keeps those at or below the smaller of the
//    two: they contain the k smallest, and they are few -- k when one slice holds the best, two to five times k
//    when the slices are alike.
// 2. Radix selection among them: the k-th smallest is found ten key bits at a time, starting below the leading
//    bits that all of them share (a 1024-bin LDS histogram per pass), until the keys at or below the prefix
//    found so far are few.  The kept keys sit in registers (at most four per thread), so a pass reads no
//    memory.  A query whose bound keeps more keys than the survivor array holds (short slices, say) runs the
//    same passes over the keys in global memory instead.
// 3. The survivors -- k of them plus the rest of the last histogram bin -- are ranked by counting in LDS
//    (sorted, when there are more than 384) and the first k written out.
// The cost grows with the number of keys, not with keys x slices x log k as a merge that ranks every key in every
// other slice does (8 slices of 100 keys: 12 us less than that merge; 32 slices of 300 keys: out of its reach),
// which is what lets a single query be split over more than eight workgroups.  Against radix passes over all
// keys in global memory, without the bound: 32 slices of 300 tied keys 21.6 -> 14.1 us, 19 slices of 1000 keys
// 85 -> 42 us, 9 slices of 100 keys 9.2 -> 8.9 us.
constexpr int kMergeSelectCap = 4096;
constexpr int kMergeSelectThreads = 1024;
constexpr int kMergeCountMax = 384;   // survivors ranked by counting; more are sorted

__global__ __launch_bounds__(kMergeSelectThreads) void ivfpq_merge_kernel(
    const key_t *__restrict__ partial, int nsplit, int k, int metric, const int64_t *__restrict__ ids,
    const int32_t *__restrict__ order, float *__restrict__ out_dist, int64_t *__restrict__ out_labels)
{
    constexpr int NT = kMergeSelectThreads;
    constexpr int kPer = kMergeSelectCap / NT;   // keys of the survivor array per thread
    static_assert(kMergeSelectCap == kPer * NT, "a thread holds its share of the survivor array in registers");
    __shared__ int hist[1024];
    __shared__ __align__(16) key_t surv[kMergeSelectCap];
    __shared__ int s_bin, s_below, s_kept;
    __shared__ key_t s_bound;
    __shared__ key_t s_min[NT / kWave], s_max[NT / kWave];
    __shared__ int s_cnt[NT / kWave];
    const int tid = threadIdx.x;
    const int64_t q = order ? order[blockIdx.x] : blockIdx.x;
    const int total = nsplit * k;
    const key_t *src = partial + q * total;

    // ---- 1. the bound, and the keys at or below it.  A query with no more keys than the survivor array holds
    // takes them into registers at once, while the first wavefront fetches the bound: one memory round trip.
    const bool small = total <= kMergeSelectCap;
    key_t mine[kPer];
#pragma unroll
    for (int j = 0; j < kPer; j++) {
        const int i = j * NT + tid;
        mine[j] = (small && i < total) ? src[i] : kEmptyKey;
    }
    if (tid < kWave) {
        // (the rank is taken as if every slice were full: a slice with fewer keys than that has kEmptyKey there,
        // which leaves the first bound alone)
        const int r = (k + nsplit - 1) / nsplit;
        key_t full_min = kEmptyKey, rank_max = 0;
        for (int j = tid; j < nsplit; j += kWave) {
            const key_t last = src[(int64_t)j * k + (k - 1)], at_r = src[(int64_t)j * k + (r - 1)];
            full_min = last < full_min ? last : full_min;
            rank_max = at_r > rank_max ? at_r : rank_max;
        }
        for (int o = 32; o > 0; o >>= 1) {
            const key_t a = __shfl_xor(full_min, o), b = __shfl_xor(rank_max, o);
            full_min = a < full_min ? a : full_min;
            rank_max = b > rank_max ? b : rank_max;
        }
        if (tid == 0) {
            s_bound = full_min < rank_max ? full_min : rank_max;
            s_kept = 0;
        }
    }
    __syncthreads();
    // every pass over the keys in global memory keeps four loads per thread in flight; fn sees every key,
    // kEmptyKey included, and is called the same number of times by every thread (it may hold ballots)
    auto visit_global = [&](auto &&fn) {
        for (int base = 0; base < total; base += NT * kPer) {
            key_t kk[kPer];
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                const int i = base + j * NT + tid;
                kk[j] = i < total ? src[i] : kEmptyKey;
            }
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                fn(kk[j]);
            }
        }
    };
    // appends the keys that a wavefront keeps to the survivor array: one LDS atomic per wavefront and call
    // (every lane calls, the same number of times)
    auto append = [&](bool keep, key_t key) {
        const unsigned long long m = __ballot(keep);
        if (m == 0) {
            return;
        }
        const int lane = tid & (kWave - 1), leader = __ffsll((long long)m) - 1;
        int base = 0;
        if (lane == leader) {
            base = atomicAdd(&s_kept, __popcll(m));
        }
        base = __shfl(base, leader);
        const int at = base + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0));
        if (keep && at < kMergeSelectCap) {
            surv[at] = key;
        }
    };
    bool in_regs = small;   // uniform over the workgroup: the rest of the selection never reads global memory
    {
        const key_t bound = s_bound;
        if (small) {
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                mine[j] = mine[j] <= bound ? mine[j] : kEmptyKey;
            }
        } else {
            visit_global([&](key_t key) { append(key != kEmptyKey && key <= bound, key); });
            __syncthreads();
            const int bounded = s_kept;
            in_regs = bounded <= kMergeSelectCap;
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                const int i = j * NT + tid;
                mine[j] = (in_regs && i < bounded) ? surv[i] : kEmptyKey;
            }
        }
    }
    auto visit = [&](auto &&fn) {
        if (in_regs) {
#pragma unroll
            for (int j = 0; j < kPer; j++) {
                fn(mine[j]);
            }
        } else {
            visit_global(fn);
        }
    };
    __syncthreads();   // the survivor array is free again: every thread has its keys

    // ---- 2. radix selection among the kept keys (all keys of the query, when the bound kept too many).  They
    // share their leading bits (sign, exponent and more): the selection starts below the common prefix of the
    // smallest and the largest
    key_t mn = kEmptyKey, mx = 0;
    int nvalid = 0;
    visit([&](key_t key) {
        if (key != kEmptyKey) {
            mn = key < mn ? key : mn;
            mx = key > mx ? key : mx;
            nvalid++;
        }
    });
    for (int o = 32; o > 0; o >>= 1) {
        const key_t omn = __shfl_xor(mn, o), omx = __shfl_xor(mx, o);
        mn = omn < mn ? omn : mn;
        mx = omx > mx ? omx : mx;
        nvalid += __shfl_xor(nvalid, o);
    }
    if ((tid & (kWave - 1)) == 0) {
        s_min[tid / kWave] = mn;
        s_max[tid / kWave] = mx;
        s_cnt[tid / kWave] = nvalid;
    }
    __syncthreads();
    nvalid = 0;
    for (int w = 0; w < NT / kWave; w++) {
        mn = s_min[w] < mn ? s_min[w] : mn;
        mx = s_max[w] > mx ? s_max[w] : mx;
        nvalid += s_cnt[w];
    }

    // Few enough to rank at once: every one of them survives.  A pass over keys in registers costs about what
    // ranking 64 more survivors does, a pass over global memory three times that.
    const int few = in_regs ? k + 64 : (k + 64 > 320 ? k + 64 : 320);
    bool all = nvalid <= k || (nvalid <= kMergeSelectCap && nvalid <= few);
    int shift = (all || mn == mx) ? 0 : 64 - __clzll((long long)(mn ^ mx));   // the keys differ below this bit
    key_t prefix = shift >= 64 ? 0 : mn >> shift;   // the bits above `shift` of the k-th smallest key
    int need = k;                                    // rank of that key among the keys that share the prefix
    while (!all && shift > 0) {
        const int bits = shift >= 10 ? 10 : shift;
        const int upper = shift;   // keys are compared with `prefix` above this bit
        shift -= bits;
        for (int i = tid; i < 1024; i += NT) {
            hist[i] = 0;
        }
        __syncthreads();
        // (tied scores put most keys of a pass into one bin: the lanes that share the first counted lane's bin
        // add once for all of them, the others one by one)
        visit([&](key_t key) {
            const bool counted = key != kEmptyKey && (upper == 64 || (key >> upper) == prefix);
            const uint32_t bin = (uint32_t)(key >> shift) & ((1u << bits) - 1u);
            const unsigned long long any = __ballot(counted);
            if (any) {
                const int leader = __ffsll((long long)any) - 1;
                const uint32_t leader_bin = (uint32_t)__shfl((int)bin, leader);
                const unsigned long long same = __ballot(counted && bin == leader_bin);
                if ((tid & (kWave - 1)) == leader) {
                    atomicAdd(&hist[leader_bin], __popcll(same));
                } else if (counted && bin != leader_bin) {
                    atomicAdd(&hist[bin], 1);
                }
            }
        });
        __syncthreads();
        if (tid < kWave) {
            // first bin whose inclusive count reaches `need`: 16 bins per lane, a wave scan over the lanes
            int part = 0;
            for (int j = 0; j < 16; j++) {
                part += hist[tid * 16 + j];
            }
            int incl = part;
#pragma unroll
            for (int o = 1; o < kWave; o <<= 1) {
                const int up = __shfl_up(incl, o);
                if (tid >= o) {
                    incl += up;
                }
            }
            const unsigned long long reach = __ballot(incl >= need);   // never empty: nvalid > k >= need
            const int owner = reach ? __ffsll((long long)reach) - 1 : kWave - 1;
            if (tid == owner) {
                int below = incl - part, bin = tid * 16;
                while (bin < tid * 16 + 15 && below + hist[bin] < need) {
                    below += hist[bin];
                    bin++;
                }
                s_bin = bin;
                s_below = below;
                s_kept = hist[bin];
            }
        }
        __syncthreads();
        prefix = (prefix << bits) | (key_t)(uint32_t)s_bin;
        need -= s_below;
        const int survivors = (k - need) + s_kept;   // keys below the prefix class + the class itself
        __syncthreads();
        if (survivors <= kMergeSelectCap && survivors <= few) {
            break;
        }
    }
    if (tid == 0) {
        s_kept = 0;
    }
    __syncthreads();
    visit([&](key_t key) { append(key != kEmptyKey && (all || shift >= 64 || (key >> shift) <= prefix), key); });
    __syncthreads();

    // ---- 3. rank the survivors
    const int kept = s_kept < kMergeSelectCap ? s_kept : kMergeSelectCap;
    const float pad = metric == kMetricL2 ? 3.402823466e+38f : -3.402823466e+38f;
    if (kept <= kMergeCountMax) {
        // rank by counting (work grows with the square of the survivors: beyond a few hundred the sort below wins).  With fewer survivors than threads, `parts` threads share a survivor: each counts over
        // its stretch of the array (neighbouring lanes read the same keys: LDS broadcasts) and adds to the
        // survivor's rank in LDS.
        const int parts = kept > 0 ? (NT / kept < 8 ? (NT / kept < 1 ? 1 : NT / kept) : 8) : 1;
        const int stretch = (kept + parts - 1) / parts;
        for (int i = tid; i < kept; i += NT) {
            hist[i] = 0;
        }
        __syncthreads();
        {
            const int e = tid / parts, part = tid - e * parts;
            if (e < kept) {
                const key_t me = surv[e];
                const int j0 = part * stretch, j1 = j0 + stretch < kept ? j0 + stretch : kept;
                int rank = 0;
                for (int j = j0; j < j1; j++) {
                    const key_t v = surv[j];
                    rank += (v < me || (v == me && j < e)) ? 1 : 0;
                }
                atomicAdd(&hist[e], rank);
            }
        }
        __syncthreads();
        for (int e = tid; e < kept; e += NT) {
            const int rank = hist[e];
            if (rank < k) {
                const key_t me = surv[e];
                const float v = key_score(me);
                out_dist[q * k + rank] = metric == kMetricL2 ? v : -v;
                out_labels[q * k + rank] = ids[key_index(me)];
            }
        }
        for (int i = kept + tid; i < k; i += NT) {
            out_dist[q * k + i] = pad;
            out_labels[q * k + i] = -1;
        }
        return;
    }
    int n2 = 512;
    while (n2 < kept) {
        n2 <<= 1;
    }
    for (int i = kept + tid; i < n2; i += NT) {
        surv[i] = kEmptyKey;
    }
    block_bitonic_sort(surv, n2, tid, NT);
    for (int i = tid; i < k; i += NT) {
        const key_t kk = i < kept ? surv[i] : kEmptyKey;
        const bool ok = kk != kEmptyKey;
        const float v = key_score(kk);
        out_dist[q * k + i] = ok ? (metric == kMetricL2 ? v : -v) : pad;
        out_labels[q * k + i] = ok ? ids[key_index(kk)] : -1;
    }
}

// Sum of the lengths of all probed lists (the number of codes the scan visits): grid-stride
// partial sums, one atomic per workgroup.
__global__ __launch_bounds__(256) void count_scanned_kernel(const int32_t *__restrict__ probes, int64_t n,
                                                            const int32_t *__restrict__ list_len, int nlist,
                                                            unsigned long long *__restrict__ out)
{
    __shared__ unsigned long long part[4];
    unsigned long long v = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int l = probes[i];
        v += (uint32_t)l < (uint32_t)nlist ? (unsigned long long)list_len[l] : 0ull;
    }
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_down(v, o);
    }
    if ((threadIdx.x & 63) == 0) {
        part[threadIdx.x >> 6] = v;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        atomicAdd(out, part[0] + part[1] + part[2] + part[3]);
    }
}

void launch_count_scanned(const int32_t *probes, int64_t n, const int32_t *list_len, int nlist, unsigned long long *out,
                          hipStream_t s)
{
    if (n == 0) {
        return;
    }
    const unsigned grid = (unsigned)std::min<int64_t>(64, (n + 255) / 256);
    hipLaunchKernelGGL(count_scanned_kernel, dim3(grid), dim3(256), 0, s, probes, n, list_len, nlist, out);
}

// ---- execution order: heaviest queries first ------------------------------------------------------
// A launch of few workgroups with very different amounts of work (skewed lists, large nprobe) ends
// with a long tail when a heavy query happens to start late.  Three small kernels order the queries
// by descending work class (work = codes to scan, 1024 classes up to max_work) with a counting sort;
// the order inside a class is whatever the atomics give -- it only decides when a workgroup runs.
constexpr int kWorkClasses = 1024;

// one wavefront per query: cls[q] and the class histogram
__global__ __launch_bounds__(256) void work_class_kernel(const int32_t *__restrict__ probes, int64_t nq, int nprobe,
                                                         const int32_t *__restrict__ list_len, int nlist,
                                                         long long max_work, int32_t *__restrict__ cls,
                                                         int32_t *__restrict__ hist)
{
    const int64_t q = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (q >= nq) {
        return;
    }
    long long w = 0;
    for (int j = lane; j < nprobe; j += 64) {
        const int l = probes[q * nprobe + j];
        w += (uint32_t)l < (uint32_t)nlist ? list_len[l] : 0;
    }
    for (int o = 32; o > 0; o >>= 1) {
        w += __shfl_xor(w, o);
    }
    if (lane == 0) {
        long long c = w * kWorkClasses / (max_work + 1);
        c = c < 0 ? 0 : (c > kWorkClasses - 1 ? kWorkClasses - 1 : c);
        cls[q] = (int32_t)c;
        atomicAdd(&hist[c], 1);
    }
}

// one workgroup: cursor[c] = queries in classes above c; the histogram is left zeroed for the next call
__global__ __launch_bounds__(kWorkClasses) void class_offsets_kernel(int32_t *__restrict__ hist,
                                                                    int32_t *__restrict__ cursor)
{
    __shared__ int32_t scan[kWorkClasses];
    const int t = threadIdx.x, c = kWorkClasses - 1 - t;   // thread 0 owns the heaviest class
    const int32_t mine = hist[c];
    hist[c] = 0;
    scan[t] = mine;
    __syncthreads();
    for (int o = 1; o < kWorkClasses; o <<= 1) {
        const int32_t add = t >= o ? scan[t - o] : 0;
        __syncthreads();
        scan[t] += add;
        __syncthreads();
    }
    cursor[c] = scan[t] - mine;
}

__global__ __launch_bounds__(256) void scatter_order_kernel(const int32_t *__restrict__ cls, int64_t nq,
                                                            int32_t *__restrict__ cursor, int32_t *__restrict__ order)
{
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q < nq) {
        order[atomicAdd(&cursor[cls[q]], 1)] = (int32_t)q;
    }
}

// ---- execution order: queries that probe the same lists side by side ---------------------------------
// Queries drawn from one cluster of the data probe nearly the same lists, and the smallest list id
// among a query's probes is then the same for most of them.  A hash of that id is the query's class,
// so the counting sort above puts such queries next to each other (with a few strangers whose hash
// collides, which does no harm: only neighbourhood in time matters, and a class is much shorter than
// the set of workgroups an XCD runs at once).  Results do not depend on the order.  (Sorting every
// query's probe list by list id as well, so that neighbours walk their common lists in the same
// sequence, was measured and is slower: 1.79 against 1.71 ms on 10000 queries x 64 lists of a 10M index.)
__global__ __launch_bounds__(256) void locality_class_kernel(const int32_t *__restrict__ probes, int64_t nq, int nprobe,
                                                             int32_t *__restrict__ cls, int32_t *__restrict__ hist)
{
    const int64_t q = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (q >= nq) {
        return;
    }
    uint32_t lowest = 0xffffffffu;   // -1 (no list) is the largest value as unsigned
    for (int j = lane; j < nprobe; j += 64) {
        const uint32_t l = (uint32_t)probes[q * nprobe + j];
        lowest = l < lowest ? l : lowest;
    }
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)lowest, o);
        lowest = other < lowest ? other : lowest;
    }
    if (lane == 0) {
        const int c = (int)((lowest * 2654435761u) >> 22);   // 1024 classes
        cls[q] = c;
        atomicAdd(&hist[c], 1);
    }
}

void launch_order_by_locality(const int32_t *probes, int64_t nq, int nprobe, int32_t *cls, int32_t *hist,
                              int32_t *cursor, int32_t *order, hipStream_t s)
{
    static_assert(kWorkClasses == 1024, "the class hash keeps ten bits");
    if (nq == 0) {
        return;
    }
    hipLaunchKernelGGL(locality_class_kernel, dim3((unsigned)((nq + 3) / 4)), dim3(256), 0, s, probes, nq, nprobe, cls,
                       hist);
    hipLaunchKernelGGL(class_offsets_kernel, dim3(1), dim3(kWorkClasses), 0, s, hist, cursor);
    hipLaunchKernelGGL(scatter_order_kernel, dim3((unsigned)((nq + 255) / 256)), dim3(256), 0, s, cls, nq, cursor, order);
}

void launch_order_by_work(const int32_t *probes, int64_t nq, int nprobe, const int32_t *list_len, int nlist,
                          long long max_work, int32_t *cls, int32_t *hist, int32_t *cursor, int32_t *order, hipStream_t s)
{
    if (nq == 0) {
        return;
    }
    hipLaunchKernelGGL(work_class_kernel, dim3((unsigned)((nq + 3) / 4)), dim3(256), 0, s, probes, nq, nprobe, list_len,
                       nlist, max_work, cls, hist);
    hipLaunchKernelGGL(class_offsets_kernel, dim3(1), dim3(kWorkClasses), 0, s, hist, cursor);
    hipLaunchKernelGGL(scatter_order_kernel, dim3((unsigned)((nq + 255) / 256)), dim3(256), 0, s, cls, nq, cursor, order);
}

// The row-layout lookups address the LUT from LDS address 0: true while the kernel declares no static LDS, which
// is asked of the loaded code object once per kernel and refused loudly otherwise.
static void require_no_static_lds(const void *kern, std::atomic<bool> &checked)
{
    if (checked.load(std::memory_order_acquire)) {
        return;
    }
    hipFuncAttributes attr{};
    IXA_HIP(hipFuncGetAttributes(&attr, kern));
    IXA_REQUIRE(attr.sharedSizeBytes == 0, kErrInner,
                "the scan kernel has %zu bytes of static LDS: its LUT would not start at LDS address 0",
                (size_t)attr.sharedSizeBytes);
    checked.store(true, std::memory_order_release);
}

template <int MT, typename LutT, int LAYOUT>
static void launch_one(const ScanParams &p, int64_t nq, size_t smem, hipStream_t s)
{
    const int64_t slots = p.xcd_chunks ? (nq + 7) / 8 * 8 : nq;
    static std::atomic<bool> lds_checked[4] = {{false}, {false}, {false}, {false}};
    if (p.shared_pool && p.waves == 16) {
        auto kern = ivfpq_scan_kernel<MT, LutT, LAYOUT, 16, true>;
        require_no_static_lds(reinterpret_cast<const void *>(kern), lds_checked[0]);
        require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        hipLaunchKernelGGL(kern, dim3((unsigned)(slots * p.nsplit)), dim3(1024), smem, s, p);
    } else if (p.shared_pool) {
        auto kern = ivfpq_scan_kernel<MT, LutT, LAYOUT, 8, true>;
        require_no_static_lds(reinterpret_cast<const void *>(kern), lds_checked[1]);
        require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        hipLaunchKernelGGL(kern, dim3((unsigned)(slots * p.nsplit)), dim3(512), smem, s, p);
    } else if (p.waves == 8) {
        auto kern = ivfpq_scan_kernel<MT, LutT, LAYOUT, 8, false>;
        require_no_static_lds(reinterpret_cast<const void *>(kern), lds_checked[2]);
        require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        hipLaunchKernelGGL(kern, dim3((unsigned)(slots * p.nsplit)), dim3(512), smem, s, p);
    } else {
        auto kern = ivfpq_scan_kernel<MT, LutT, LAYOUT, 4, false>;
        require_no_static_lds(reinterpret_cast<const void *>(kern), lds_checked[3]);
        require_dynamic_lds(reinterpret_cast<const void *>(kern), smem);
        hipLaunchKernelGGL(kern, dim3((unsigned)(slots * p.nsplit)), dim3(256), smem, s, p);
    }
}

template <typename LutT>
static void dispatch_m(const ScanParams &p, int64_t nq, size_t smem, hipStream_t s)
{
    if (p.code_layout == 2) {
        if constexpr (sizeof(LutT) == 4) {
            if (p.M == 48) {
                return launch_one<48, LutT, 2>(p, nq, smem, s);
            }
        }
        fail(kErrInner, "xor48 code layout needs M = 48 and an fp32 LUT");
    }
    if (p.code_layout == 1) {
        switch (p.M) {
            case 32: return launch_one<32, LutT, 1>(p, nq, smem, s);
            case 64: return launch_one<64, LutT, 1>(p, nq, smem, s);
            case 96: return launch_one<96, LutT, 1>(p, nq, smem, s);
            default: fail(kErrInner, "rot32 code layout needs M in {32, 64, 96}, got %d", p.M);
        }
    }
    switch (p.M) {
        // every sub-quantizer count of the reference's own envelope (2, 4, 8, 16, 32:
        // FR/ascend/impl/AscendIndexIVFPQImpl.cpp:130-140) has a kernel with compile-time M
        case 2: return launch_one<2, LutT, 0>(p, nq, smem, s);
        case 4: return launch_one<4, LutT, 0>(p, nq, smem, s);
        case 8: return launch_one<8, LutT, 0>(p, nq, smem, s);
        case 16: return launch_one<16, LutT, 0>(p, nq, smem, s);
        case 32: return launch_one<32, LutT, 0>(p, nq, smem, s);
        case 48: return launch_one<48, LutT, 0>(p, nq, smem, s);
        case 64: return launch_one<64, LutT, 0>(p, nq, smem, s);
        case 96: return launch_one<96, LutT, 0>(p, nq, smem, s);
        default: return launch_one<0, LutT, 0>(p, nq, smem, s);
    }
}

static size_t plan_with_waves(ScanParams &p, int waves, bool shared)
{
    size_t lut_bytes = (size_t)p.M * 256 * (p.lut_fp16 ? 2 : 4);
    if (p.code_layout == 1 && p.lut_fp16) {
        lut_bytes += 64;   // the upper half of the last row lies in the row after it (rot32_half_slot)
    }
    if (p.code_layout == 2) {
        lut_bytes = (size_t)64 * 256 * 4;
    }
    p.waves = waves;
    p.shared_pool = shared ? 1 : 0;
    p.cap = shared ? block_pool_capacity(p.k, waves) : wave_pool_capacity(p.k);
    p.merge_n = shared ? p.cap : waves * p.cap;
    p.table_n = (p.nprobe + p.nsplit - 1) / p.nsplit;
    size_t off = round_up((int64_t)lut_bytes, 16);
    p.off_query = (int)off;
    off += round_up((int64_t)p.d * 4, 16);
    p.off_pools = (int)off;
    off += (size_t)p.merge_n * sizeof(key_t);   // also the merge array of the epilogue
    p.off_merge = p.off_pools;
    p.off_table = (int)off;
    off += round_up((int64_t)p.table_n * 12, 16);
    p.off_hist = (int)off;
    off += shared ? 4096 : 0;
    p.off_misc = (int)off;
    // share[W] + counts[W] + BlockPoolCtl.  (Sized for eight waves this region ended 32 bytes short with
    // sixteen: harmless while the plan's total is rounded up by the LDS allocation granule, a workgroup
    // that never finishes when the total is an exact multiple of it.)
    off += (size_t)round_up(8 * waves + (int64_t)sizeof(BlockPoolCtl), 64);
    return off;
}

// Wavefronts one CU can hold with this plan (LDS- and thread-limited; 160 KB, 2048 threads).
static int resident_waves(size_t smem, int waves)
{
    const int by_lds = (int)(160 * 1024 / smem), by_threads = 2048 / (waves * 64);
    return std::min(by_lds, by_threads) * waves;
}

// Private pools with eight wavefronts per workgroup when three such workgroups fit the 160 KB of
// a CU; otherwise whichever of {private x 8, private x 4, shared x 8, shared x 16} keeps most
// wavefronts resident (earlier in that list on ties).  Private pools of more than 256 keys (k > 128) then
// give way to one shared pool of eight wavefronts: with them every wavefront keeps and compacts a top-k of
// its own out of an eighth of the candidates (10M x 128, M 32, nprobe 64, 10000 queries: k = 160 scans in
// 3.07 ms with private pools and 2.63 ms with the shared one, k = 256 in 3.48 / 2.71 ms, k = 100 -- 256-key
// pools -- in 1.68 / 2.61 ms; one query over 32 lists of 9800 four-byte codes, k = 300: 209 / 99 us).
static size_t plan_scan_by_residency(ScanParams &p);

size_t plan_scan(ScanParams &p)
{
    const ScanParams asked = p;
    const size_t smem = plan_scan_by_residency(p);
    if (!p.shared_pool && p.cap > 256 && block_pool_capacity(asked.k, 8) <= 8 * 8 * kWave) {
        ScanParams q = asked;
        const size_t shared_smem = plan_with_waves(q, 8, true);
        if (shared_smem <= 160 * 1024) {
            p = q;
            return shared_smem;
        }
    }
    return smem;
}

static size_t plan_scan_by_residency(ScanParams &p)
{
    ScanParams best = p;
    size_t best_smem = plan_with_waves(best, 8, false);
    if (best_smem * 3 <= 160 * 1024) {
        p = best;
        return best_smem;
    }
    int best_waves = best_smem <= 160 * 1024 ? resident_waves(best_smem, 8) : 0;
    ScanParams smallest = best;   // reported when nothing fits
    size_t smallest_smem = best_smem;
    const struct {
        int waves;
        bool shared;
    } alts[] = {{4, false}, {8, true}, {16, true}};
    for (const auto &alt : alts) {
        if (alt.shared && block_pool_capacity(p.k, alt.waves) > (alt.waves >= 16 ? 4 : 8) * alt.waves * kWave) {
            continue;
        }
        ScanParams q = p;
        const size_t smem = plan_with_waves(q, alt.waves, alt.shared);
        // a shared-pool workgroup keeps its CU to itself: those kernels need more than the 64
        // registers per lane that a second resident workgroup would leave them
        const int rw = smem <= 160 * 1024 ? (alt.shared ? alt.waves : resident_waves(smem, alt.waves)) : 0;
        if (rw > best_waves) {
            best = q;
            best_smem = smem;
            best_waves = rw;
        }
        if (smem < smallest_smem) {
            smallest = q;
            smallest_smem = smem;
        }
    }
    if (best_waves == 0) {
        p = smallest;
        return smallest_smem;
    }
    p = best;
    return best_smem;
}

// The LDS plan of a launch as plain numbers (host only: no device is touched).  waves = 0 lets plan_scan()
// choose; otherwise the plan for that workgroup size and pool kind is returned as it would be laid out.
size_t scan_lds_plan(int d, int M, int lut_fp16, int code_layout, int nprobe, int nsplit, int k, int waves,
                     int shared_pool, ScanParams *out, int *ctl_bytes)
{
    ScanParams p{};
    p.d = d;
    p.M = M;
    p.lut_fp16 = lut_fp16;
    p.code_layout = code_layout;
    p.nprobe = nprobe;
    p.nsplit = nsplit;
    p.k = k;
    const size_t smem = waves == 0 ? plan_scan(p) : plan_with_waves(p, waves, shared_pool != 0);
    *out = p;
    *ctl_bytes = (int)sizeof(BlockPoolCtl);
    return smem;
}

void launch_scan(ScanParams p, int64_t nq, hipStream_t s)
{
    if (nq == 0) {
        return;
    }
    p.nq = nq;
    const size_t smem = plan_scan(p);
    IXA_REQUIRE(smem <= 160 * 1024, kErrInvalidParam,
                "IVFPQ scan needs at least %zu bytes of LDS (M=%d, k=%d, %s LUT); the limit is 163840", smem, p.M, p.k,
                p.lut_fp16 ? "fp16" : "fp32");
    IXA_REQUIRE(nq * p.nsplit < ((int64_t)1 << 31), kErrInvalidParam, "scan grid too large");
    IXA_REQUIRE(p.nsplit == 1 || p.partial != nullptr, kErrInner, "a split scan needs a buffer for its partial lists");
    if (p.lut_fp16) {
        dispatch_m<__half>(p, nq, smem, s);
    } else {
        dispatch_m<float>(p, nq, smem, s);
    }
    if (p.nsplit > 1) {
        hipLaunchKernelGGL(ivfpq_merge_kernel, dim3((unsigned)nq), dim3(kMergeSelectThreads), 0, s, p.partial,
                           p.nsplit, p.k, p.metric, p.ids, p.order, p.out_dist, p.out_labels);
    }
}

}  // namespace ixa
