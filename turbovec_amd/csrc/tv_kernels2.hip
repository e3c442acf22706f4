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
// fetches the same entry of all QL queries, and the bytes are accumulated as
// packed 16-bit lanes that are widened every 256 byte-groups -- the same flush
// period the reference uses, which makes the classic epilogue's per-batch
// fma(scale, f32(batch_sum), fa) reproducible exactly.
// ===========================================================================

template <int QL> struct LutWord;
template <> struct LutWord<1> { typedef uint8_t type; };
template <> struct LutWord<2> { typedef uint16_t type; };
template <> struct LutWord<4> { typedef uint32_t type; };

template <int QL, int U, int MODE, bool LUT_LDS>
__global__ __launch_bounds__(kScanThreads) void k_scan_lut(ScanArgs a) {
    typedef typename LutWord<QL>::type word_t;
    constexpr bool LISTS = MODE == kModeLists, DUMP = MODE == kModeDump, APPEND = MODE == kModeAppend;
    extern __shared__ __align__(16) uint8_t smem[];
    const int nch = a.nch, k = a.k;
    const size_t lut_bytes = LUT_LDS ? size_t(nch) * 1024 * QL : 0;
    float *sct = reinterpret_cast<float *>(smem + lut_bytes);            // [4 waves][QL][32]
    float *ls = sct + 4 * QL * 32;
    uint32_t *li = reinterpret_cast<uint32_t *>(ls + (LISTS ? k * kScanThreads : 0));
    int *stau = reinterpret_cast<int *>(li + (LISTS ? k * kScanThreads : 0));
    const int tid = threadIdx.x;

    if (LUT_LDS) {
        // interleave: entry e of query qq -> smem[e*QL + qq]
        for (int w = tid; w < nch * 256; w += kScanThreads) {
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
    const word_t *lut = LUT_LDS ? reinterpret_cast<const word_t *>(smem) : reinterpret_cast<const word_t *>(a.tables);

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
    const uint32_t total_waves = gridDim.x * (kScanThreads / 64);
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
        for (int u = 0; u < U; ++u) buf[u] = codes[(size_t(j) * step * nch + u) * 64];
    }
    while (j < j_end) {
        const uint32_t nj_live = live_from(j + total_waves);
        const uint32_t b = j * step;
        uint32_t total[QL];
        float fa[QL];
#pragma unroll
        for (int qq = 0; qq < QL; ++qq) { total[qq] = 0; fa[qq] = qb[qq]; }
        uint32_t accE = 0, accO = 0;
        for (int c0 = 0; c0 < nch; c0 += U) {
            uint4 cur[U];
#pragma unroll
            for (int u = 0; u < U; ++u) cur[u] = buf[u];
            if (c0 + U < nch) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = codes[(size_t(b) * nch + c0 + U + u) * 64];
            } else if (nj_live < j_end) {
#pragma unroll
                for (int u = 0; u < U; ++u) buf[u] = codes[(size_t(nj_live) * step * nch + u) * 64];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u;
                const uint32_t x[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
                const int g0 = c * 32 + 16 * h;
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const uint32_t byte = (x[j >> 2] >> (8 * (j & 3))) & 0xffu;
                    const int row = (g0 + j) * 32;
                    const uint32_t vh = lut[row + (byte >> 4)];
                    const uint32_t vl = lut[row + 16 + (byte & 15u)];
                    if (QL == 1) {
                        accE += vh + vl;
                    } else {
                        accE += (vh & 0x00ff00ffu) + (vl & 0x00ff00ffu);
                        accO += ((vh >> 8) & 0x00ff00ffu) + ((vl >> 8) & 0x00ff00ffu);
                    }
                }
                if ((c & 7) == 7 || c == nch - 1) {  // end of a 256-group batch (search.rs:529-531)
                    uint32_t part[QL];
                    if (QL == 1) part[0] = accE;
                    if (QL == 2) { part[0] = accE; part[1] = accO; }
                    if (QL == 4) { part[0] = accE & 0xffffu; part[1] = accO & 0xffffu; part[2] = accE >> 16; part[3] = accO >> 16; }
                    accE = 0; accO = 0;
#pragma unroll
                    for (int qq = 0; qq < QL; ++qq) {
                        part[qq] += __shfl_xor(int(part[qq]), 32);
                        total[qq] += part[qq];
                        fa[qq] = fmaf(qs[qq], float(part[qq]), fa[qq]);  // search.rs:577-580
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
            score[qq] = a.classic ? fa[qq] * vs : ((float(int(total[qq])) * qs[qq]) + qb[qq]) * vs;
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
                                if (list_offer(L, ls, li, kScanThreads, tid, k, s, slot) && a.share_tau) {
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
        const size_t total_threads = size_t(gridDim.x) * kScanThreads;
        const size_t gt = size_t(blockIdx.x) * kScanThreads + tid;
        a.part_cnt[gt] = L.cnt;
        for (int e = 0; e < L.cnt; ++e) {
            a.part_scores[size_t(e) * total_threads + gt] = ls[e * kScanThreads + tid];
            a.part_idx[size_t(e) * total_threads + gt] = li[e * kScanThreads + tid];
        }
    }
}

static constexpr size_t kLdsBudgetL = 160 * 1024;

static size_t lut_lds_bytes(int nch, int k, int ql, bool no_lists) {
    const size_t lists = no_lists ? 0 : size_t(k) * kScanThreads * 8;
    return size_t(nch) * 1024 * ql + size_t(4) * ql * 32 * 4 + lists + kQTile * sizeof(int);
}

int lut_tile_queries(int nch, int k) {
    for (int ql = 4; ql >= 1; ql >>= 1)
        if (lut_lds_bytes(nch, k, ql, false) <= kLdsBudgetL) return ql;
    return 1;  // table read from global memory
}

template <typename K>
static hipError_t allow_lds2(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               int(bytes));
}

int lut_launch_ql(int nch, int k, int nq_tile) {
    int ql = lut_tile_queries(nch, k);
    while (ql > 1 && ql / 2 >= nq_tile) ql >>= 1;
    return ql;
}

// One launch serves a.nq_tile <= lut_tile_queries(nch, k) queries.
hipError_t launch_scan_lut(const ScanArgs &a, int grid, int mode, hipStream_t s) {
    const bool dump = mode != kModeLists;   // no list storage in LDS
    const int kk = a.k;                     // the tile width is chosen for the list pass of the same search
    const int ql = lut_launch_ql(a.nch, kk, a.nq_tile);
    const bool in_lds = lut_lds_bytes(a.nch, kk, ql, dump) <= kLdsBudgetL;
    const size_t lds = in_lds ? lut_lds_bytes(a.nch, kk, ql, dump)
                              : lut_lds_bytes(0, kk, 1, dump);
    hipError_t e = hipSuccess;
#define TV_LAUNCH_L(QL, U, D, W)                                                                 \
    do {                                                                                         \
        e = allow_lds2(k_scan_lut<QL, U, D, W>, lds);                                            \
        if (e != hipSuccess) return e;                                                           \
        hipLaunchKernelGGL((k_scan_lut<QL, U, D, W>), dim3(grid), dim3(kScanThreads), lds, s, a); \
    } while (0)
#define TV_PICK_M(QL, U, W)                                                                      \
    do {                                                                                         \
        if (mode == kModeDump) TV_LAUNCH_L(QL, U, kModeDump, W);                                 \
        else if (mode == kModeAppend) TV_LAUNCH_L(QL, U, kModeAppend, W);                        \
        else TV_LAUNCH_L(QL, U, kModeLists, W);                                                  \
    } while (0)
#define TV_PICK_L(QL, U) TV_PICK_M(QL, U, true)
    const int u = a.nch % 2 == 0 ? 2 : 1;
    if (!in_lds) {
        if (u == 2) TV_PICK_M(1, 2, false); else TV_PICK_M(1, 1, false);
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
