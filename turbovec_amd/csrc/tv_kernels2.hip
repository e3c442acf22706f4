// Scan for the u8-LUT score modes and the exact top-k selection used when k is
// too large for the per-lane lists.  Compiled with -ffp-contract=off.
#include <cfloat>

#include "tv_device.h"
#include "tv_internal.h"

namespace tv {

// ===========================================================================
// Scan, score modes L: per-query u8 tables, integer sums of table lookups
// (turbovec/src/search.rs:3113-3128 is the definition; the production kernels
// are :467-670, :697-984, :1071-1339).  QL queries share one pass: their
// tables are interleaved entry-major in LDS so that one QL-byte LDS read
// fetches the same entry of all QL queries.  The two reads of a code byte are
// added bytewise (entries are at most 127, so no byte carries) and each
// query's byte is peeled into its own 32-bit sum with one v_dot4_u32_u8
// against a one-hot constant.  Sums are flushed every 256 byte-groups -- the
// reference's period -- which makes the classic epilogue's per-batch
// fma(scale, f32(batch_sum), fa) reproducible exactly.  Append-mode launches
// use 1024-thread workgroups: one copy of the tables in LDS then serves four
// waves per SIMD, which is what hides the LDS and HBM latencies.
// ===========================================================================

typedef uint32_t lut_u32x2 __attribute__((ext_vector_type(2)));

// base + byte E of packed, in one instruction (sub-dword operand select).
template <int E>
__device__ __forceinline__ uint32_t add_byte(uint32_t base, uint32_t packed) {
    uint32_t r;
    if (E == 0) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 1) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 2) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 3) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(base), "v"(packed));
    return r;
}

// The m-th A operand (16 bytes) out of a lane's 16 looked-up table words.
template <int QL, typename W>
__device__ __forceinline__ v4i lut_a_operand(const W (&w)[16], int m);
template <>
__device__ __forceinline__ v4i lut_a_operand<4, uint32_t>(const uint32_t (&w)[16], int m) {
    return v4i{int(w[4 * m]), int(w[4 * m + 1]), int(w[4 * m + 2]), int(w[4 * m + 3])};
}
template <>
__device__ __forceinline__ v4i lut_a_operand<8, lut_u32x2>(const lut_u32x2 (&w)[16], int m) {
    return v4i{int(w[2 * m].x), int(w[2 * m].y), int(w[2 * m + 1].x), int(w[2 * m + 1].y)};
}
template <>
__device__ __forceinline__ v4i lut_a_operand<1, uint8_t>(const uint8_t (&)[16], int) { return v4i{0, 0, 0, 0}; }
template <>
__device__ __forceinline__ v4i lut_a_operand<2, uint16_t>(const uint16_t (&)[16], int) { return v4i{0, 0, 0, 0}; }

template <typename F>
__device__ __forceinline__ void static_for4(F &&f) { f(IntC<0>{}); f(IntC<1>{}); f(IntC<2>{}); f(IntC<3>{}); }

template <int QL> struct LutWord;
template <> struct LutWord<1> { typedef uint8_t type; };
template <> struct LutWord<2> { typedef uint16_t type; };
template <> struct LutWord<4> { typedef uint32_t type; };
template <> struct LutWord<8> { typedef lut_u32x2 type; };

// acc[q] += byte q of (vh + vl), bytewise sums never carrying (entries <= 127).
template <int QL> struct LutAcc;
template <> struct LutAcc<1> {
    static __device__ __forceinline__ void add(uint32_t (&acc)[1], uint8_t vh, uint8_t vl) { acc[0] += uint32_t(vh) + uint32_t(vl); }
};
template <> struct LutAcc<2> {
    static __device__ __forceinline__ void add(uint32_t (&acc)[2], uint16_t vh, uint16_t vl) {
        const uint32_t s = uint32_t(vh) + uint32_t(vl);
        acc[0] = __builtin_amdgcn_udot4(s, 0x00000001u, acc[0], false);
        acc[1] = __builtin_amdgcn_udot4(s, 0x00000100u, acc[1], false);
    }
};
template <> struct LutAcc<4> {
    static __device__ __forceinline__ void add(uint32_t (&acc)[4], uint32_t vh, uint32_t vl) {
        const uint32_t s = vh + vl;
        acc[0] = __builtin_amdgcn_udot4(s, 0x00000001u, acc[0], false);
        acc[1] = __builtin_amdgcn_udot4(s, 0x00000100u, acc[1], false);
        acc[2] = __builtin_amdgcn_udot4(s, 0x00010000u, acc[2], false);
        acc[3] = __builtin_amdgcn_udot4(s, 0x01000000u, acc[3], false);
    }
};
template <> struct LutAcc<8> {
    static __device__ __forceinline__ void add(uint32_t (&acc)[8], lut_u32x2 vh, lut_u32x2 vl) {
        const uint32_t s0 = vh.x + vl.x, s1 = vh.y + vl.y;
        acc[0] = __builtin_amdgcn_udot4(s0, 0x00000001u, acc[0], false);
        acc[1] = __builtin_amdgcn_udot4(s0, 0x00000100u, acc[1], false);
        acc[2] = __builtin_amdgcn_udot4(s0, 0x00010000u, acc[2], false);
        acc[3] = __builtin_amdgcn_udot4(s0, 0x01000000u, acc[3], false);
        acc[4] = __builtin_amdgcn_udot4(s1, 0x00000001u, acc[4], false);
        acc[5] = __builtin_amdgcn_udot4(s1, 0x00000100u, acc[5], false);
        acc[6] = __builtin_amdgcn_udot4(s1, 0x00010000u, acc[6], false);
        acc[7] = __builtin_amdgcn_udot4(s1, 0x01000000u, acc[7], false);
    }
};

template <int QL, int U, int MODE, bool LUT_LDS, int THREADS>
__global__ __launch_bounds__(THREADS) void k_scan_lut(ScanArgs a) {
    typedef typename LutWord<QL>::type word_t;
    constexpr bool LISTS = MODE == kModeLists, DUMP = MODE == kModeDump, APPEND = MODE == kModeAppend;
    extern __shared__ __align__(16) uint8_t smem[];
    if (APPEND && launch_switched_off(a.run_if)) return;
    const int nch = a.nch, k = a.k;
    const size_t lut_bytes = LUT_LDS ? size_t(nch) * 1024 * QL : 0;
    float *sct = reinterpret_cast<float *>(smem + lut_bytes);            // [waves][QL][32]
    float *ls = sct + (THREADS / 64) * QL * 32;
    uint32_t *li = reinterpret_cast<uint32_t *>(ls + (LISTS ? k * THREADS : 0));
    int *stau = reinterpret_cast<int *>(li + (LISTS ? k * THREADS : 0));
    const int tid = threadIdx.x;

    if (LUT_LDS) {
        // interleave: entry e of query qq -> smem[e*QL + qq]
        for (int w = tid; w < nch * 256; w += THREADS) {
            uint32_t v[QL];
#pragma unroll
            for (int qq = 0; qq < QL; ++qq)
                v[qq] = reinterpret_cast<const uint32_t *>(a.tables + size_t(qq) * nch * 1024)[w];
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
#pragma unroll
                for (int qq = 0; qq < QL; ++qq) smem[(size_t(w) * 4 + e4) * QL + qq] = uint8_t(v[qq] >> (8 * e4));
            }
        }
    }
    if (LISTS && tid < kQTile) stau[tid] = tid < QL ? a.gtau[tid] : kTauInit;
    uint32_t *scnt = reinterpret_cast<uint32_t *>(stau);  // append mode: candidates per query of this workgroup
    if (APPEND && tid < kQTile) scnt[tid] = 0u;
    __syncthreads();
    // With whole-dword table words (4 or 8 queries) the per-query sums are taken by the matrix
    // unit: a lane's looked-up words are an A operand as they are (row = its vector, 16 bytes =
    // a few groups x QL queries), and B[k][n] = 1 where byte k belongs to query n adds them up
    // per query in 32-bit integers while the vector ALU moves on to the next addresses.
    constexpr bool MF = LUT_LDS && (QL == 4 || QL == 8);
    // 16x16x64: a lane's 16 bytes are row (lane % 16) of k-block (lane / 16).  Lanes 0-15 and 32-47
    // hold vectors 0-15 (the two halves of a chunk's groups), lanes 16-31 and 48-63 vectors 16-31:
    // the one-hot B sends the odd k-blocks to a second set of QL output columns, so that one
    // instruction sums 64 bytes for each of 16 rows and no column is idle at 8 queries.
    v4i bsel = {0, 0, 0, 0};
    {
        const int n = threadIdx.x & 15, kb = (threadIdx.x >> 4) & 3;
        const bool mine = n < 2 * QL && (n / QL) == (kb & 1);
        const int qn = n % QL;
        if (QL == 4) { const int w = mine ? int(1u << (8 * qn)) : 0; bsel = v4i{w, w, w, w}; }
        if (QL == 8) {
            const int w0 = mine && qn < 4 ? int(1u << (8 * qn)) : 0, w1 = mine && qn >= 4 ? int(1u << (8 * (qn - 4))) : 0;
            bsel = v4i{w0, w1, w0, w1};
        }
    }
    const word_t *lut = LUT_LDS ? reinterpret_cast<const word_t *>(smem) : reinterpret_cast<const word_t *>(a.tables);
    // the tables' address inside LDS as a plain number: entry addresses are then formed with integer
    // adds and dereferenced as LDS pointers, with the per-byte row offsets riding in the read's offset field
    typedef const __attribute__((address_space(3))) word_t lds_word_t;
    const uint32_t lds_lut_addr = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem));

    const int lane = tid & 63, wave = tid >> 6;
    const int vi = lane & 31, h = lane >> 5;
    float qs[QL], qb[QL];
#pragma unroll
    for (int qq = 0; qq < QL; ++qq) {
        qs[qq] = qq < a.nq_tile ? a.qscale[qq] : 0.0f;
        qb[qq] = qq < a.nq_tile ? a.qbias[qq] : 0.0f;
    }
    // list ownership: lane l folds query l % QL over `per` vectors of each block
    constexpr int per = QL * 32 >= 64 ? QL * 32 / 64 : 1;
    const int oq = lane % QL, vg = lane / QL;
    const bool owner = oq < a.nq_tile && vg * per < 32;
    const float tau_fixed = APPEND ? (owner ? order_unkey(a.gtau[oq]) : __int_as_float(0x7fc00000)) : 0.0f;

    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;
    const uint32_t total_waves = gridDim.x * (THREADS / 64);
    const uint32_t gw = wave * gridDim.x + blockIdx.x;  // consecutive blocks go to different workgroups
    const uint32_t j_begin = gw, j_end = nj;   // round-robin over the grid's waves

    LaneList L{0, 0.0f, 0u, 0};
    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes) + lane;
    float *my_sct = sct + wave * QL * 32;

    auto live_from = [&](uint32_t j) -> uint32_t {
        if (a.mask == nullptr) return j;
        while (j < j_end) {
            const uint32_t b = j * step;
            const uint64_t w = a.mask[b >> 1];
            if (uint32_t(w >> ((b & 1) * 32)) != 0u) break;
            j += total_waves;
        }
        return j;
    };

    uint32_t j = live_from(j_begin);
    uint4 buf[U];
    if (j < j_end) {
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(j) * step * nch + u) * 64]);
    }
    while (j < j_end) {
        const uint32_t nj_live = live_from(j + total_waves);
        const uint32_t b = j * step;
        uint32_t total[QL];
        float fa[QL];
#pragma unroll
        for (int qq = 0; qq < QL; ++qq) { total[qq] = 0; fa[qq] = qb[qq]; }
        uint32_t acc[QL];
#pragma unroll
        for (int qq = 0; qq < QL; ++qq) acc[qq] = 0;
        v4i macc = {0, 0, 0, 0}, macc2 = {0, 0, 0, 0};   // two chains, so that dependent MFMAs do not queue
        word_t wh[16], wl[16];
        // The scalar definition (search.rs:3113-3128): score = bias, then for every byte group in
        // order score += scale * hi entry, score += scale * lo entry, each a separate f32 multiply
        // and add.  One query per launch; a vector's groups alternate between its two lanes in
        // runs of 16, and the running sum is handed from one to the other after each run.
        const bool scalar = QL == 1 && a.classic == 2;
        float chain = qb[0];
        for (int c0 = 0; c0 < nch; c0 += U) {
            uint4 cur[U];
#pragma unroll
            for (int u = 0; u < U; ++u) cur[u] = buf[u];
            if (c0 + U < nch) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(b) * nch + c0 + U + u) * 64]);
            } else if (nj_live < j_end) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(nj_live) * step * nch + u) * 64]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u;
                const uint32_t x[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
                // Byte offsets of the entries inside their 16-entry sub-tables, four code bytes at a
                // time: nibble * sizeof(word) still fits a byte, so one shift and one mask prepare
                // four of them and a byte-select add forms each LDS address.
                constexpr int kSh = QL == 1 ? 0 : QL == 2 ? 1 : QL == 4 ? 2 : 3;
                const uint8_t *gbase = reinterpret_cast<const uint8_t *>(lut);
                const uint32_t row_off = uint32_t(c * 32 + 16 * h) * 32 * QL + (LUT_LDS ? lds_lut_addr : 0u);
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t plo = (x[d] << kSh) & (0x0f0f0f0fu << kSh);
                    const uint32_t phi = (x[d] >> (4 - kSh)) & (0x0f0f0f0fu << kSh);
                    static_for4([&](auto ec) {
                        constexpr int e = decltype(ec)::value;
                        const int j = d * 4 + e;
                        word_t vh, vl;
                        if (LUT_LDS) {
                            vh = *reinterpret_cast<lds_word_t *>(add_byte<e>(row_off, phi) + j * 32 * QL);
                            vl = *reinterpret_cast<lds_word_t *>(add_byte<e>(row_off, plo) + (j * 32 + 16) * QL);
                        } else {
                            vh = *reinterpret_cast<const word_t *>(gbase + add_byte<e>(row_off, phi) + j * 32 * QL);
                            vl = *reinterpret_cast<const word_t *>(gbase + add_byte<e>(row_off, plo) + (j * 32 + 16) * QL);
                        }
                        if (MF || (QL == 1 && scalar)) { wh[j] = vh; wl[j] = vl; }
                        if (!MF) LutAcc<QL>::add(acc, vh, vl);
                    });
                }
                if constexpr (QL == 1) {
                    if (scalar) {
                        const int g0 = c * 32;
                        auto run16 = [&](float t, int gfirst) {
#pragma unroll
                            for (int jj = 0; jj < 16; ++jj) {
                                if (gfirst + jj < a.n_groups) {
                                    t = t + qs[0] * float(uint32_t(wh[jj]));
                                    t = t + qs[0] * float(uint32_t(wl[jj]));
                                }
                            }
                            return t;
                        };
                        if (h == 0) chain = run16(chain, g0);
                        chain = __shfl(chain, vi);            // the first half's sum, to both lanes of the vector
                        if (h == 1) chain = run16(chain, g0 + 16);
                        chain = __shfl(chain, vi + 32);       // and the second half's, back
                    }
                }
                if (MF) {
                    // 16 bytes of a lane = WPA groups x QL queries; the one-hot B sums them per query
                    constexpr int WPA = 16 / QL;   // words per A operand
#pragma unroll
                    for (int m = 0; m < 16 / WPA; ++m) {
                        macc = __builtin_amdgcn_mfma_i32_16x16x64_i8(lut_a_operand<QL>(wh, m), bsel, macc, 0, 0, 0);
                        macc2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(lut_a_operand<QL>(wl, m), bsel, macc2, 0, 0, 0);
                    }
                }
                if ((c & 7) == 7 || c == nch - 1) {  // end of a 256-group batch (search.rs:529-531)
                    if (MF) {
                        // lane l holds output column l % 16 (query n % QL of vector half n / QL), rows
                        // 4 * (l / 16) .. + 3: hand the sums to the lanes of their vectors through the
                        // wave's scratch rows
                        int *xch = reinterpret_cast<int *>(my_sct);
                        const int on = lane & 15;
                        if (on < 2 * QL) {
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                xch[(on % QL) * 32 + 16 * (on / QL) + 4 * (lane >> 4) + r] = macc[r] + macc2[r];
                        }
                        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
                        __builtin_amdgcn_wave_barrier();
#pragma unroll
                        for (int qq = 0; qq < QL; ++qq) acc[qq] = uint32_t(xch[qq * 32 + vi]);
                        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
                        __builtin_amdgcn_wave_barrier();
                        macc = v4i{0, 0, 0, 0};
                        macc2 = v4i{0, 0, 0, 0};
                    }
#pragma unroll
                    for (int qq = 0; qq < QL; ++qq) {
                        const uint32_t part = MF ? acc[qq] : acc[qq] + uint32_t(__shfl_xor(int(acc[qq]), 32));
                        acc[qq] = 0;
                        total[qq] += part;
                        fa[qq] = fmaf(qs[qq], float(part), fa[qq]);  // search.rs:577-580
                    }
                }
            }
        }

        const uint32_t slot0 = b * 32u;
        uint32_t mw = 0xffffffffu;
        if (a.mask != nullptr) mw = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
        const float vs = a.scales[slot0 + vi];
        float score[QL];
#pragma unroll
        for (int qq = 0; qq < QL; ++qq) {
            // classic: fa * vec_scale; u32: ((f32(acc) * scale) + bias) * vec_scale (search.rs:1174-1177)
            score[qq] = a.classic == 1 ? fa[qq] * vs : ((float(int(total[qq])) * qs[qq]) + qb[qq]) * vs;
            if (QL == 1 && a.classic == 2) score[qq] = chain * vs;
        }
        if (DUMP) {
            const uint32_t slot = slot0 + vi;
            if (h == 0 && slot < a.n) {
#pragma unroll
                for (int qq = 0; qq < QL; ++qq) {
                    if (qq < a.nq_tile) {
                        const size_t o = size_t(qq) * a.n + slot;
                        if (a.acc_out) a.acc_out[o] = int(total[qq]);
                        if (a.score_out) a.score_out[o] = ((mw >> vi) & 1u) ? score[qq] : __int_as_float(0x7fc00000);
                    }
                }
            }
        } else {
            if (h == 0) {
#pragma unroll
                for (int qq = 0; qq < QL; ++qq) my_sct[qq * 32 + vi] = score[qq];
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            __builtin_amdgcn_wave_barrier();
            if (APPEND) {
#pragma unroll
                for (int e = 0; e < per; ++e) {
                    const int i = (vg * per + e) & 31;
                    const float s = my_sct[oq * 32 + i];
                    const uint32_t slot = slot0 + i;
                    if (s >= tau_fixed && slot < a.n && ((mw >> i) & 1u)) {
                        const uint32_t pos = atomicAdd(&scnt[oq], 1u);
                        if (pos < kSegCap)
                            a.cand[(size_t(oq) * a.seg_stride + blockIdx.x) * kSegCap + pos] = sort_key(s, slot);
                    }
                }
            } else {
                if (a.share_tau && (j & 3u) == 0u && lane < QL) atomicMax(&stau[lane], a.gtau[lane]);
                if (owner) {
                    const float tau = order_unkey(stau[oq]);
#pragma unroll
                    for (int e = 0; e < per; ++e) {
                        const int i = vg * per + e;
                        const float s = my_sct[oq * 32 + i];
                        const uint32_t slot = slot0 + i;
                        if (s >= tau && (L.cnt < k || ranks_before(s, slot, L.worst_s, L.worst_i))) {
                            if (slot < a.n && ((mw >> i) & 1u)) {
                                if (list_offer(L, ls, li, THREADS, tid, k, s, slot) && a.share_tau) {
                                    const int key = order_key(L.worst_s);
                                    if (atomicMax(&stau[oq], key) < key) atomicMax(&a.gtau[oq], key);
                                }
                            }
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            __builtin_amdgcn_wave_barrier();
        }
        j = nj_live;
    }

    if (APPEND) {
        __syncthreads();
        if (tid < a.nq_tile) a.cand_cnt[size_t(tid) * a.seg_stride + blockIdx.x] = scnt[tid];
    }
    if (LISTS) {
        const size_t total_threads = size_t(gridDim.x) * THREADS;
        const size_t gt = size_t(blockIdx.x) * THREADS + tid;
        a.part_cnt[gt] = L.cnt;
        for (int e = 0; e < L.cnt; ++e) {
            a.part_scores[size_t(e) * total_threads + gt] = ls[e * THREADS + tid];
            a.part_idx[size_t(e) * total_threads + gt] = li[e * THREADS + tid];
        }
    }
}

// ===========================================================================
// Single-query scan over byte tables, score modes L, append mode.
//
// With one query the two nibble tables of a byte-group (16 entries each) are first folded
// into one 256-entry table per code byte in LDS -- entry b = lut[hi nibble of b] +
// lut[16 + lo nibble of b], at most 254, so still a byte -- and the scan then makes ONE LDS
// read per code byte instead of two, addressed by the raw code byte (no nibble split).  The
// integer sums are those of the two-read walk (turbovec/src/search.rs:3113-3128), term for
// term, so the epilogues reproduce the reference's floats as before.  A byte table takes 256
// bytes per byte-group (96 KiB at 1536 dimensions and 2 bits); rows too long for that get byte
// tables for their first n_bt chunks and keep the two nibble reads for the rest (19 of 24
// chunks at 1536 dimensions and 4 bits).
// ===========================================================================
constexpr int kLutBtThreads = 1024;

template <int U>
__global__ __launch_bounds__(kLutBtThreads) void k_scan_lut_bt(ScanArgs a, int n_bt) {
    extern __shared__ __align__(16) uint8_t smem[];
    if (launch_switched_off(a.run_if)) return;
    const int nch = a.nch;
    uint8_t *bt = smem;                                                   // [n_bt * 32][256]
    uint8_t *nt = smem + size_t(n_bt) * 8192;                             // [(nch - n_bt) * 32][32]: the nibble tables as built
    uint32_t *scnt = reinterpret_cast<uint32_t *>(nt + size_t(nch - n_bt) * 1024);
    const int tid = threadIdx.x;
    // fold: four entries (one dword) per step
    for (int w = tid; w < n_bt * 32 * 64; w += kLutBtThreads) {
        const int g = w >> 6, b0 = (w & 63) * 4;
        const uint8_t *row = a.tables + size_t(g) * 32;
        const uint32_t hi = row[b0 >> 4];
        uint32_t v = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) v |= (hi + uint32_t(row[16 + ((b0 + e) & 15)])) << (8 * e);
        reinterpret_cast<uint32_t *>(bt)[w] = v;
    }
    for (int w = tid; w < (nch - n_bt) * 256; w += kLutBtThreads)
        reinterpret_cast<uint32_t *>(nt)[w] = reinterpret_cast<const uint32_t *>(a.tables + size_t(n_bt) * 1024)[w];
    if (tid == 0) *scnt = 0u;
    __syncthreads();
    typedef const __attribute__((address_space(3))) uint8_t lds_byte_t;
    const uint32_t lds_bt = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem));
    const uint32_t lds_nt = lds_bt + uint32_t(n_bt) * 8192;

    const int lane = tid & 63, wave = tid >> 6;
    const int vi = lane & 31, h = lane >> 5;
    const float qs = a.qscale[0], qb = a.qbias[0];
    const float tau = order_unkey(a.gtau[0]);
    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;
    const uint32_t total_waves = gridDim.x * (kLutBtThreads / 64);
    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes) + lane;

    auto live_from = [&](uint32_t j) -> uint32_t {
        if (a.mask == nullptr) return j;
        while (j < nj) {
            const uint32_t b = j * step;
            if (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) != 0u) break;
            j += total_waves;
        }
        return j;
    };

    uint32_t j = live_from(wave * gridDim.x + blockIdx.x);   // consecutive blocks go to different workgroups
    uint4 buf[U];
    if (j < nj) {
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(j) * step * nch + u) * 64]);
    }
    while (j < nj) {
        const uint32_t nj_live = live_from(j + total_waves);
        const uint32_t b = j * step;
        uint32_t total = 0, acc = 0;
        float fa = qb;
        for (int c0 = 0; c0 < nch; c0 += U) {
            uint4 cur[U];
#pragma unroll
            for (int u = 0; u < U; ++u) cur[u] = buf[u];
            if (c0 + U < nch) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(b) * nch + c0 + U + u) * 64]);
            } else if (nj_live < nj) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(nj_live) * step * nch + u) * 64]);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u;
                const uint32_t x[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
                if (c < n_bt) {
                    const uint32_t row_off = lds_bt + uint32_t(c * 32 + 16 * h) * 256;
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        static_for4([&](auto ec) {
                            constexpr int e = decltype(ec)::value;
                            acc += uint32_t(*reinterpret_cast<lds_byte_t *>(add_byte<e>(row_off, x[d]) + (d * 4 + e) * 256));
                        });
                    }
                } else {
                    const uint32_t row_off = lds_nt + uint32_t((c - n_bt) * 32 + 16 * h) * 32;
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        const uint32_t plo = x[d] & 0x0f0f0f0fu, phi = (x[d] >> 4) & 0x0f0f0f0fu;
                        static_for4([&](auto ec) {
                            constexpr int e = decltype(ec)::value;
                            acc += uint32_t(*reinterpret_cast<lds_byte_t *>(add_byte<e>(row_off, phi) + (d * 4 + e) * 32));
                            acc += uint32_t(*reinterpret_cast<lds_byte_t *>(add_byte<e>(row_off, plo) + (d * 4 + e) * 32 + 16));
                        });
                    }
                }
                if ((c & 7) == 7 || c == nch - 1) {  // end of a 256-group batch (search.rs:529-531)
                    const uint32_t part = acc + uint32_t(__shfl_xor(int(acc), 32));
                    acc = 0;
                    total += part;
                    fa = fmaf(qs, float(part), fa);   // search.rs:577-580
                }
            }
        }
        const uint32_t slot0 = b * 32u;
        uint32_t mw = 0xffffffffu;
        if (a.mask != nullptr) mw = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
        const uint32_t slot = slot0 + uint32_t(vi);
        const bool allowed = h == 0 && slot < a.n && ((mw >> vi) & 1u);
        float sc = 0.0f;
        if (allowed) {
            const float vs = a.scales[slot];
            // classic: fa * vec_scale; u32: ((f32(acc) * scale) + bias) * vec_scale (search.rs:1174-1177)
            sc = a.classic == 1 ? fa * vs : ((float(int(total)) * qs) + qb) * vs;
        }
        if (a.best_of_block) {
            // A first sampling level without a floor: the block's best allowed row (score order, then
            // the lower slot: the larger sort key), one candidate per block -- a real score of a real
            // row, so the k-th best of these is a floor k scanned rows reach.
            uint64_t key = allowed && sc == sc ? sort_key(sc, slot) : 0ull;
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                const uint32_t ohi = uint32_t(__shfl_xor(int(uint32_t(key >> 32)), d));
                const uint32_t olo = uint32_t(__shfl_xor(int(uint32_t(key)), d));
                const uint64_t o = (uint64_t(ohi) << 32) | olo;
                key = o > key ? o : key;
            }
            if (lane == 0 && key != 0ull) {
                const uint32_t pos = atomicAdd(scnt, 1u);
                if (pos < kSegCap) a.cand[size_t(blockIdx.x) * kSegCap + pos] = key;
            }
        } else if (allowed && sc >= tau) {
            const uint32_t pos = atomicAdd(scnt, 1u);
            if (pos < kSegCap) a.cand[size_t(blockIdx.x) * kSegCap + pos] = sort_key(sc, slot);
        }
        j = nj_live;
    }
    __syncthreads();
    if (tid == 0) a.cand_cnt[blockIdx.x] = *scnt;
}

// Chunks of a row that get byte tables when `budget` bytes of LDS are available, and the bytes used.
static int lut_bt_chunks(int nch, size_t budget) {
    const size_t fixed = size_t(nch) * 1024 + 64;
    if (budget <= fixed) return 0;
    const size_t n = (budget - fixed) / (8192 - 1024);
    return int(n < size_t(nch) ? n : size_t(nch));
}
static size_t lut_bt_lds_bytes(int nch, int n_bt) { return size_t(n_bt) * 8192 + size_t(nch - n_bt) * 1024 + 64; }

static constexpr size_t kLdsBudgetL = 160 * 1024;

static size_t lut_lds_bytes(int nch, int k, int ql, bool no_lists, int threads) {
    const size_t lists = no_lists ? 0 : size_t(k) * threads * 8;
    return size_t(nch) * 1024 * ql + size_t(threads / 64) * ql * 32 * 4 + lists + kQTile * sizeof(int);
}

constexpr int kLutListThreads = kScanThreads;   // exact paths: per-lane lists or dense dump
constexpr int kLutAppendThreads = 1024;         // sample-then-filter scans

// Queries one list- or dump-mode launch serves.
int lut_tile_queries(int nch, int k) {
    for (int ql = 4; ql >= 1; ql >>= 1)
        if (lut_lds_bytes(nch, k, ql, false, kLutListThreads) <= kLdsBudgetL) return ql;
    return 1;  // table read from global memory
}

// Queries one append-mode launch serves (tables of all of them resident in LDS, one copy per CU).
int lut_append_queries(int nch) {
    for (int ql = 8; ql >= 1; ql >>= 1)
        if (lut_lds_bytes(nch, 0, ql, true, kLutAppendThreads) <= kLdsBudgetL) return ql;
    return 1;
}

static int lut_cus = 256;   // compute units of the device the last grid was sized for

int lut_append_grid(int device, int nch) {
    hipDeviceProp_t prop;
    int cus = 256;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        cus = prop.multiProcessorCount;
    lut_cus = cus;
    const size_t lds = lut_lds_bytes(nch, 0, lut_append_queries(nch), true, kLutAppendThreads);
    return cus * (lds * 2 <= kLdsBudgetL ? 2 : 1);   // at most 2048 threads per CU
}

template <typename K>
static hipError_t allow_lds2(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               int(bytes));
}

// Whether a single query's append-mode launch on a grid of `grid` workgroups goes to the byte-table
// scan (which also serves a first level without floors, ScanArgs::best_of_block).
bool lut_single_uses_byte_tables(int nch, int grid) {
    const int n_bt = lut_bt_chunks(nch, grid > lut_cus ? kLdsBudgetL / 2 : kLdsBudgetL);
    return n_bt * 2 >= nch;
}

int lut_launch_ql(int nch, int k, int nq_tile) {
    int ql = lut_tile_queries(nch, k);
    while (ql > 1 && ql / 2 >= nq_tile) ql >>= 1;
    return ql;
}

// One launch serves a.nq_tile queries: at most lut_append_queries(nch) in append mode,
// lut_tile_queries(nch, k) otherwise.
hipError_t launch_scan_lut(const ScanArgs &a, int grid, int mode, hipStream_t s) {
    const bool append = mode == kModeAppend;
    const bool scalar = a.classic == 2;     // the chain of float adds: one query per launch, nibble tables
    if (scalar && a.nq_tile != 1) return hipErrorInvalidValue;
    if (append && a.nq_tile == 1 && !scalar) {
        // one query: byte tables for as many chunks as fit, one LDS read per code byte there
        const int n_bt = lut_bt_chunks(a.nch, grid > lut_cus ? kLdsBudgetL / 2 : kLdsBudgetL);
        if (n_bt * 2 >= a.nch) {
            const size_t lds = lut_bt_lds_bytes(a.nch, n_bt);
            hipError_t e = hipSuccess;
#define TV_LAUNCH_BT(U)                                                                          \
            do {                                                                                 \
                e = allow_lds2(k_scan_lut_bt<U>, lds);                                           \
                if (e != hipSuccess) return e;                                                   \
                hipLaunchKernelGGL(k_scan_lut_bt<U>, dim3(grid), dim3(kLutBtThreads), lds, s, a, n_bt); \
            } while (0)
            if (a.nch % 4 == 0) TV_LAUNCH_BT(4);
            else if (a.nch % 2 == 0) TV_LAUNCH_BT(2);
            else TV_LAUNCH_BT(1);
#undef TV_LAUNCH_BT
            return hipGetLastError();
        }
    }
    const bool dump = mode != kModeLists;   // no list storage in LDS
    const int kk = a.k;                     // the tile width is chosen for the list pass of the same search
    const int threads = append ? kLutAppendThreads : kLutListThreads;
    int ql = scalar ? 1 : append ? lut_append_queries(a.nch) : lut_tile_queries(a.nch, kk);
    while (ql > 1 && ql / 2 >= a.nq_tile) ql >>= 1;
    const bool in_lds = lut_lds_bytes(a.nch, kk, ql, dump, threads) <= kLdsBudgetL;
    const size_t lds = in_lds ? lut_lds_bytes(a.nch, kk, ql, dump, threads)
                              : lut_lds_bytes(0, kk, 1, dump, threads);
    hipError_t e = hipSuccess;
#define TV_LAUNCH_L(QL, U, D, W, T)                                                              \
    do {                                                                                         \
        e = allow_lds2(k_scan_lut<QL, U, D, W, T>, lds);                                         \
        if (e != hipSuccess) return e;                                                           \
        hipLaunchKernelGGL((k_scan_lut<QL, U, D, W, T>), dim3(grid), dim3(T), lds, s, a);        \
    } while (0)
#define TV_PICK_M(QL, U, W)                                                                      \
    do {                                                                                         \
        if (mode == kModeDump) TV_LAUNCH_L(QL, U, kModeDump, W, kLutListThreads);                \
        else if (mode == kModeAppend) TV_LAUNCH_L(QL, U, kModeAppend, W, kLutAppendThreads);     \
        else TV_LAUNCH_L(QL, U, kModeLists, W, kLutListThreads);                                 \
    } while (0)
#define TV_PICK_L(QL, U) TV_PICK_M(QL, U, true)
    const int u = a.nch % 2 == 0 ? 2 : 1;
    if (!in_lds) {
        if (u == 2) TV_PICK_M(1, 2, false); else TV_PICK_M(1, 1, false);
    } else if (ql == 8) {
        if (!append) return hipErrorInvalidValue;
        if (u == 2) TV_LAUNCH_L(8, 2, kModeAppend, true, kLutAppendThreads);
        else TV_LAUNCH_L(8, 1, kModeAppend, true, kLutAppendThreads);
    } else if (ql == 4) { if (u == 2) TV_PICK_L(4, 2); else TV_PICK_L(4, 1); }
    else if (ql == 2) { if (u == 2) TV_PICK_L(2, 2); else TV_PICK_L(2, 1); }
    else { if (u == 2) TV_PICK_L(1, 2); else TV_PICK_L(1, 1); }
#undef TV_PICK_L
#undef TV_PICK_M
#undef TV_LAUNCH_L
    return hipGetLastError();
}

// ===========================================================================
// Exact top-k of dense score rows (k beyond the per-lane lists): radix select
// on the unique 64-bit keys (score order, then lower slot), gather, sort.
// State per query lives behind its 2048-bin histogram:
//   hist[2048] = prefix low, [2049] = prefix high, [2050] = remaining,
//   [2051] = gather cursor.
// ===========================================================================

constexpr int kSelStride = 4096;

__global__ void k_sel_init(uint32_t *hist, uint64_t *tmp, uint32_t k_eff, uint32_t sort_n) {
    uint32_t *h = hist + size_t(blockIdx.y) * kSelStride;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < 2048) h[i] = 0;
    if (i == 0) { h[2048] = 0; h[2049] = 0; h[2050] = k_eff; h[2051] = 0; }
    if (i >= k_eff && i < sort_n) tmp[size_t(blockIdx.y) * sort_n + i] = 0;
}

__global__ __launch_bounds__(256) void k_sel_hist(const float *__restrict__ scores, size_t n, uint32_t *hist,
                                                  int shift, int digit_bits) {
    __shared__ uint32_t lh[2048];
    uint32_t *h = hist + size_t(blockIdx.y) * kSelStride;
    for (int i = threadIdx.x; i < 2048; i += 256) lh[i] = 0;
    __syncthreads();
    const uint64_t prefix = (uint64_t(h[2049]) << 32) | h[2048];
    const int upper = shift + digit_bits;
    const uint32_t dmask = (1u << digit_bits) - 1;
    const float *row = scores + size_t(blockIdx.y) * n;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256) {
        const float s = row[i];
        if (s != s) continue;
        const uint64_t key = sort_key(s, uint32_t(i));
        if (upper < 64 && ((key ^ prefix) >> upper) != 0) continue;
        atomicAdd(&lh[uint32_t(key >> shift) & dmask], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 2048; i += 256)
        if (lh[i]) atomicAdd(&h[i], lh[i]);
}

__global__ __launch_bounds__(256) void k_sel_pick(uint32_t *hist, int shift, int digit_bits) {
    uint32_t *h = hist + size_t(blockIdx.x) * kSelStride;
    __shared__ uint32_t chosen;
    if (threadIdx.x == 0) {
        uint32_t remaining = h[2050];
        int d = (1 << digit_bits) - 1;
        for (; d > 0; --d) {
            if (h[d] >= remaining) break;
            remaining -= h[d];
        }
        const uint64_t prefix = ((uint64_t(h[2049]) << 32) | h[2048]) | (uint64_t(uint32_t(d)) << shift);
        h[2048] = uint32_t(prefix);
        h[2049] = uint32_t(prefix >> 32);
        h[2050] = remaining;
        chosen = uint32_t(d);
    }
    __syncthreads();
    (void)chosen;
    for (int i = threadIdx.x; i < 2048; i += 256) h[i] = 0;
}

__global__ __launch_bounds__(256) void k_sel_gather(const float *__restrict__ scores, size_t n, uint32_t *hist,
                                                    uint64_t *tmp, uint32_t k_eff, uint32_t sort_n) {
    uint32_t *h = hist + size_t(blockIdx.y) * kSelStride;
    const uint64_t kth = (uint64_t(h[2049]) << 32) | h[2048];
    const float *row = scores + size_t(blockIdx.y) * n;
    for (size_t i = size_t(blockIdx.x) * 256 + threadIdx.x; i < n; i += size_t(gridDim.x) * 256) {
        const float s = row[i];
        if (s != s) continue;
        const uint64_t key = sort_key(s, uint32_t(i));
        if (key >= kth) {
            const uint32_t pos = atomicAdd(&h[2051], 1u);
            if (pos < k_eff) tmp[size_t(blockIdx.y) * sort_n + pos] = key;
        }
    }
}

__global__ __launch_bounds__(256) void k_sel_bitonic(uint64_t *tmp, uint32_t sort_n, uint32_t size, uint32_t stride) {
    uint64_t *keys = tmp + size_t(blockIdx.y) * sort_n;
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= sort_n / 2) return;
    const uint32_t lo = 2 * i - (i & (stride - 1));
    const uint32_t hi = lo + stride;
    const bool desc = (lo & size) == 0;
    const uint64_t x = keys[lo], y = keys[hi];
    if ((x < y) == desc) { keys[lo] = y; keys[hi] = x; }
}

__global__ __launch_bounds__(256) void k_sel_emit(const uint64_t *tmp, uint32_t sort_n, uint32_t k_eff,
                                                  float *out_scores, int64_t *out_idx) {
    const uint32_t j = blockIdx.x * 256 + threadIdx.x;
    if (j >= k_eff) return;
    float s; uint32_t idx;
    sort_unkey(tmp[size_t(blockIdx.y) * sort_n + j], s, idx);
    out_scores[size_t(blockIdx.y) * k_eff + j] = s;
    out_idx[size_t(blockIdx.y) * k_eff + j] = int64_t(idx);
}

size_t select_tmp_keys(size_t k_eff) {
    size_t p = 2;
    while (p < k_eff) p <<= 1;
    return p;
}

hipError_t launch_select_topk(const float *d_scores, size_t n, int nq_tile, size_t k_eff, uint64_t *d_keys_tmp,
                              uint32_t *d_hist, float *out_scores, int64_t *out_idx, hipStream_t s) {
    if (nq_tile == 0 || k_eff == 0) return hipSuccess;
    const uint32_t sort_n = uint32_t(select_tmp_keys(k_eff));
    const unsigned init_blocks = unsigned((std::max<size_t>(sort_n, 2048) + 255) / 256);
    hipLaunchKernelGGL(k_sel_init, dim3(init_blocks, nq_tile), dim3(256), 0, s, d_hist, d_keys_tmp, uint32_t(k_eff),
                       sort_n);
    const unsigned slices = unsigned(std::min<size_t>(1024, (n + 256 * 8 - 1) / (256 * 8)));
    static const int shifts[6] = {53, 42, 31, 20, 9, 0};
    static const int widths[6] = {11, 11, 11, 11, 11, 9};
    for (int p = 0; p < 6; ++p) {
        hipLaunchKernelGGL(k_sel_hist, dim3(slices, nq_tile), dim3(256), 0, s, d_scores, n, d_hist, shifts[p],
                           widths[p]);
        hipLaunchKernelGGL(k_sel_pick, dim3(nq_tile), dim3(256), 0, s, d_hist, shifts[p], widths[p]);
    }
    hipLaunchKernelGGL(k_sel_gather, dim3(slices, nq_tile), dim3(256), 0, s, d_scores, n, d_hist, d_keys_tmp,
                       uint32_t(k_eff), sort_n);
    for (uint32_t size = 2; size <= sort_n; size <<= 1)
        for (uint32_t stride = size >> 1; stride > 0; stride >>= 1)
            hipLaunchKernelGGL(k_sel_bitonic, dim3((sort_n / 2 + 255) / 256, nq_tile), dim3(256), 0, s, d_keys_tmp,
                               sort_n, size, stride);
    hipLaunchKernelGGL(k_sel_emit, dim3(unsigned((k_eff + 255) / 256), nq_tile), dim3(256), 0, s, d_keys_tmp, sort_n,
                       uint32_t(k_eff), out_scores, out_idx);
    return hipGetLastError();
}

}  // namespace tv
