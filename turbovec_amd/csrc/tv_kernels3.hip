// Wide batched scan, score mode P, append mode: one pass over the codes serves
// every query of the chunk (up to 1024), not one group of tiles per pass.
//
// A wave decodes its 32-vector block once into registers -- the int8 A operands
// of all its chunks, 8 VGPRs per chunk -- and keeps them there while the
// workgroup walks the query tiles: each tile's weights stream from L2 into LDS
// in half-tile slices through a ring of LDS slots, requested four slices ahead
// by direct-to-LDS loads that use no registers; a slice is NCH/2 chunks, i.e. NCH MFMAs per wave against B
// operands read from LDS.  The nibble decode and the HBM read of the codes are
// paid once per block instead of once per 96 queries, which leaves the matrix
// unit as the bound: 2 * 32 * 32 * 32 * NCH * 2 int8 operations per (block, tile).
//
// Integers and float epilogue are those of k_scan_p4 (turbovec/src/search.rs:
// 1392-1567, 1519-1524); only the order in which (block, tile) pairs are visited
// differs, and the candidate segments make the result independent of it.
#include "tv_device.h"
#include "tv_internal.h"

namespace tv {

constexpr int kWideThreads = 512;    // 8 waves, 2 per SIMD: one wave's epilogue and decode run under the other's MFMAs
constexpr int kWideWaves = kWideThreads / 64;
constexpr int kWideRing = 5;         // LDS slots of half a tile each; kWideRing - 1 slices are requested ahead

// 16 bytes per lane from global memory (uniform base + 16 * lane) straight into LDS at
// lds_addr + 16 * lane (lds_addr uniform over the wave).  Counted by the vector-memory counter
// like a load.  Uniform bases live in scalar registers: the kernel has no vector register to spare.
__device__ __forceinline__ void dma16_to_lds(uint32_t lds_addr, const void *sbase, uint32_t lane16) {
    const uint32_t u = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(u), "v"(lane16), "s"(sbase) : "memory");
}

// 16 bytes per lane from uniform base + 16 * lane into registers, invisible to the compiler's
// wait-count bookkeeping (wait_vm<N> on the destination is the matching wait).
__device__ __forceinline__ void load16_async_s(u32x4 &dst, const void *sbase, uint32_t lane16) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(dst) : "v"(lane16), "s"(sbase));
}

// 16 bytes of LDS per lane, requested without telling the compiler's wait-count bookkeeping;
// lds_wait<N> on the destination holds until at most N younger LDS requests are outstanding.
template <int OFF>
__device__ __forceinline__ void lds_read16_async(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF));
}
template <int N>
__device__ __forceinline__ void lds_wait(v4i &r) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N));
}

struct WideQuery {          // per query, in LDS
    float qs, qb, tau;      // tau is NaN for the padding queries of the last tile: nothing passes
    uint32_t cnt;           // candidates this workgroup appended
};

template <int NCH, int NB>
__global__ __launch_bounds__(kWideThreads, 2) void k_scan_p4_wide(ScanArgs a) {
    static_assert(NCH % 2 == 0, "a slice is half of the chunks");
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int kSlice = NCH * 1024;                      // half a tile: NCH/2 chunks x (low, high) x 1 KiB
    constexpr int kPieces = NCH / kWideWaves;               // direct-to-LDS loads per wave and slice ...
    constexpr int kExtra = NCH % kWideWaves;                // ... plus one more in the first kExtra waves
    constexpr int kAhead = kWideRing - 1;
    const int nq = a.nq_tile;
    const int nt = (nq + kQTile - 1) / kQTile;
    const int nq_pad = nt * kQTile;
    const int n_slices = 2 * nt;                            // per pass over the tiles; the host guarantees >= kAhead
    WideQuery *sq = reinterpret_cast<WideQuery *>(smem + kWideRing * kSlice);
    float *s_vs = reinterpret_cast<float *>(sq + nq_pad);   // [waves][32]: row scales, NaN where not allowed
    uint32_t *snext = reinterpret_cast<uint32_t *>(s_vs + kWideWaves * 32);
    const uint32_t lds_b = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qn = lane & 31, h = lane >> 5;
    const uint32_t lane16 = uint32_t(lane) * 16;
    for (int q = tid; q < nq_pad; q += kWideThreads) {
        const bool act = q < nq;
        sq[q].qs = act ? a.qscale[q] : 0.0f;
        sq[q].qb = act ? a.qbias[q] : 0.0f;
        sq[q].tau = act ? order_unkey(a.gtau[q]) : __int_as_float(0x7fc00000);
        sq[q].cnt = 0u;
    }
    if (tid == 0) *snext = 0u;
    __syncthreads();

    const uint32_t t0 = a.lv[0], t1 = a.lv[1], t2 = a.lv[2], t3 = a.lv[3];
    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;

    // next live block of this workgroup (blocks m * gridDim.x + blockIdx.x), claimed wave by wave
    auto claim = [&]() -> uint32_t {
        for (;;) {
            uint32_t m = 0;
            if (lane == 0) m = atomicAdd(snext, 1u);
            m = uint32_t(__builtin_amdgcn_readfirstlane(int(m)));
            const uint32_t j = m * gridDim.x + blockIdx.x;
            if (j >= nj || a.mask == nullptr) return j;
            const uint32_t b = j * step;
            if (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) != 0u) return j;
        }
    };

    // The weights are one periodic stream of slices (slice s = half s & 1 of tile s >> 1, kSlice
    // contiguous bytes; after the last tile the first follows again for the next round of blocks).
    // Stream position g lives in ring slot g % kWideRing and is requested kAhead positions early, so
    // behind the slice being consumed exactly (kAhead - 1) * kPieces of this wave's requests are
    // younger -- the count its wait leaves outstanding (waves below kExtra request one piece more).
    int req_slice = 0, req_slot = 0;                        // next stream position to request
    auto request_next = [&]() {
        const uint8_t *src = a.tables + size_t(req_slice) * kSlice + size_t(wave) * 1024;
        const uint32_t dst = lds_b + uint32_t(req_slot) * kSlice + uint32_t(wave) * 1024;
#pragma unroll
        for (int p = 0; p < kPieces; ++p)
            dma16_to_lds(dst + uint32_t(p) * (kWideWaves * 1024), src + size_t(p) * (kWideWaves * 1024), lane16);
        if (kExtra != 0 && wave < kExtra)
            dma16_to_lds(dst + uint32_t(kPieces) * (kWideWaves * 1024), src + size_t(kPieces) * (kWideWaves * 1024), lane16);
        req_slice = req_slice + 1 == n_slices ? 0 : req_slice + 1;
        req_slot = req_slot + 1 == kWideRing ? 0 : req_slot + 1;
    };
    for (int i = 0; i < kAhead; ++i) request_next();
    int use_slot = 0;                                       // ring slot of the slice consumed next

    // Wait for the slice in use_slot, let everyone catch up, refill the slot freed by the previous
    // slice, and return the consumed slice's B-operand address for this lane.
    auto next_slice = [&]() -> uint32_t {
        if (kExtra != 0 && wave < kExtra)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kAhead - 1) * (kPieces + 1)) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kAhead - 1) * kPieces) : "memory");
        __syncthreads();
        request_next();
        const uint32_t bp = lds_b + uint32_t(use_slot) * kSlice + lane16;
        use_slot = use_slot + 1 == kWideRing ? 0 : use_slot + 1;
        return bp;
    };

    v4i alo[NCH], ahi[NCH];
    v16i acc;
    // The NCH MFMAs of one slice.  MFMA m takes chunk HALF * NCH/2 + m/2 (low nibbles for even m,
    // high for odd) against the 1 KiB of weights at m * 1024, which come through NB registers
    // requested NB MFMAs ahead.
    auto slice_mfmas = [&](auto half, uint32_t baddr) {
        constexpr int c0 = decltype(half)::value * (NCH / 2);
        v4i w[NB];
        static_for<NB>([&](auto mm) { lds_read16_async<decltype(mm)::value * 1024>(w[decltype(mm)::value], baddr); });
        static_for<NCH>([&](auto mm) {
            constexpr int m = decltype(mm)::value;
            constexpr int younger = NCH - 1 - m < NB - 1 ? NCH - 1 - m : NB - 1;
            lds_wait<younger>(w[m % NB]);
            if constexpr ((m & 1) == 0)
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo[c0 + m / 2], w[m % NB], acc, 0, 0, 0);
            else
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi[c0 + m / 2], w[m % NB], acc, 0, 0, 0);
            if constexpr (m + NB < NCH) lds_read16_async<(m + NB) * 1024>(w[m % NB], baddr);
        });
    };

    // Waves w and w + 4 share a SIMD and would otherwise reach their epilogues together with the
    // MFMA pipe idle: the upper four score a tile one slice later, before the first MFMAs of
    // the next tile, while the lower four already run theirs.
    const bool late = wave >= kWideWaves / 2;

    for (;;) {
        // ---- block phase: claim, load, decode into registers ----
        const uint32_t j = claim();
        const bool has = j < nj;
        const uint32_t b = has ? j * step : 0u;
        if (has) {
            // two bursts of NCH/2 chunks: the raw codes of a burst and the operands decoded so far
            // have to fit the register file together
            const uint8_t *p = a.codes + size_t(b) * NCH * 1024;
            static_for<2>([&](auto hh) {
                constexpr int c0 = decltype(hh)::value * (NCH / 2);
                u32x4 raw[NCH / 2];
                static_for<NCH / 2>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    load16_async_s(raw[c], p + size_t(c0 + c) * 1024, lane16);
                });
                static_for<NCH / 2>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    wait_vm<NCH / 2 - 1 - c>(raw[c]);
                    const uint32_t x[4] = {raw[c].x, raw[c].y, raw[c].z, raw[c].w};
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        alo[c0 + c][d] = int(levels_of(x[d] & 0x0f0f0f0fu, t0, t1, t2, t3));
                        ahi[c0 + c][d] = int(levels_of((x[d] >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3));
                    }
                });
            });
            if (lane < 32) {
                const uint32_t slot = b * 32u + uint32_t(lane);
                bool ok = slot < a.n;
                if (ok && a.mask != nullptr) ok = (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) >> lane) & 1u;
                s_vs[wave * 32 + lane] = ok ? a.scales[slot] : __int_as_float(0x7fc00000);
            }
        }
        if (!__syncthreads_or(has ? 1 : 0)) break;

        // ---- tile phase ----
        // Scores of tile t for this wave's block; lane owns query t*32 + qn and rows
        // 8*(r/4) + 4*h + r%4 (search.rs:1519-1524).  Candidates are rare, so one pass only
        // tests the 16 scores and a second, entered by few waves, appends the ones that pass.
        auto epilogue = [&](int t) {
            const int q = t * kQTile + qn;
            const float4 qp = *reinterpret_cast<const float4 *>(sq + q);
            const float qs = qp.x, qb = qp.y, tau = qp.z;
            const float4 *vs4 = reinterpret_cast<const float4 *>(s_vs + wave * 32 + 4 * h);
            bool any = false;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 v = vs4[2 * g];
                any |= fmaf(float(acc[4 * g + 0]), qs, qb) * v.x >= tau;
                any |= fmaf(float(acc[4 * g + 1]), qs, qb) * v.y >= tau;
                any |= fmaf(float(acc[4 * g + 2]), qs, qb) * v.z >= tau;
                any |= fmaf(float(acc[4 * g + 3]), qs, qb) * v.w >= tau;
            }
            if (any) {
                const float *vs = s_vs + wave * 32 + 4 * h;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = 8 * (r >> 2) + (r & 3);
                    const float s = fmaf(float(acc[r]), qs, qb) * vs[i];
                    if (s >= tau) {
                        const uint32_t pos = atomicAdd(&sq[q].cnt, 1u);
                        if (pos < kSegCap)
                            a.cand[(size_t(q) * a.seg_stride + blockIdx.x) * kSegCap + pos] =
                                sort_key(s, b * 32u + uint32_t(i + 4 * h));
                    }
                }
            }
        };
        for (int t = 0;; ++t) {
            uint32_t b0 = 0;
            if (t < nt) b0 = next_slice();
            if (has && late && t > 0) epilogue(t - 1);
            if (t == nt) break;
            if (has) {
                acc = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                slice_mfmas(IntC<0>{}, b0);
            }
            const uint32_t b1 = next_slice();
            if (has) {
                slice_mfmas(IntC<1>{}, b1);
                if (!late) epilogue(t);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // requests still in flight write this workgroup's LDS
    __syncthreads();
    for (int q = tid; q < nq; q += kWideThreads) a.cand_cnt[size_t(q) * a.seg_stride + blockIdx.x] = sq[q].cnt;
}

// Matrix-unit probe: the wide kernel's MFMA loop alone -- A operands resident in registers,
// B operands read from LDS, pseudo-random bytes in both (operand toggling sets the power
// the clock is managed against) -- with no HBM traffic, no barriers and no epilogue.  Its rate
// is what this loop shape can sustain on the chip at hand; the nominal peak assumes the top clock.
__global__ __launch_bounds__(kWideThreads, 2) void k_probe_mfma(int iters, uint32_t *sink) {
    constexpr int NCH = 24, NB = 2;
    extern __shared__ __align__(16) uint8_t smem[];
    for (uint32_t i = threadIdx.x; i < NCH * 1024 / 4; i += kWideThreads)
        reinterpret_cast<uint32_t *>(smem)[i] = (i * 2654435761u) ^ ((i * 40503u) << 13) ^ ((i >> 3) * 97u);
    __syncthreads();
    const uint32_t baddr = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem)) +
                           (threadIdx.x & 63) * 16;
    v4i alo[NCH], ahi[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        uint32_t x = (threadIdx.x * 64 + c) * 2654435761u;
        alo[c] = v4i{int(x), int(x * 31u + 7u), int((x * 131u) ^ 0x5bd1e995u), int(x * 1664525u + 1013904223u)};
        x ^= 0x9e3779b9u;
        ahi[c] = v4i{int(x * 17u), int(x * 31u + 9u), int((x * 137u) ^ 0x5bd1e995u), int(x * 22695477u + 1u)};
    }
    v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
        static_for<2>([&](auto hh) {
            constexpr int c0 = decltype(hh)::value * (NCH / 2);
            v4i w[NB];
            static_for<NB>([&](auto mm) { lds_read16_async<decltype(mm)::value * 1024>(w[decltype(mm)::value], baddr); });
            static_for<NCH>([&](auto mm) {
                constexpr int m = decltype(mm)::value;
                constexpr int younger = NCH - 1 - m < NB - 1 ? NCH - 1 - m : NB - 1;
                lds_wait<younger>(w[m % NB]);
                if constexpr ((m & 1) == 0)
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo[c0 + m / 2], w[m % NB], acc, 0, 0, 0);
                else
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi[c0 + m / 2], w[m % NB], acc, 0, 0, 0);
                if constexpr (m + NB < NCH) lds_read16_async<(m + NB) * 1024>(w[m % NB], baddr);
            });
        });
    }
    uint32_t x = 0;
#pragma unroll
    for (int r = 0; r < 16; ++r) x ^= uint32_t(acc[r]);
    if (x == 0x9e3779b9u && iters < 0) sink[0] = x;   // keeps the loop alive; never taken
}

// One launch of the probe on every CU; *ops = int8 operations (2 per multiply-add) it performs.
hipError_t launch_probe_mfma(int device, int iters, uint32_t *sink, double *ops, hipStream_t s) {
    const int grid = wide_grid_blocks(device);
    hipLaunchKernelGGL(k_probe_mfma, dim3(grid), dim3(kWideThreads), 24 * 1024, s, iters, sink);
    if (ops) *ops = double(grid) * kWideWaves * double(iters) * 48.0 * 65536.0;
    return hipGetLastError();
}

// Smallest chunk of queries the wide kernel is the faster one for (measured against the
// tile-group kernels on 4-bit indexes of 1024, 1280 and 1536 dimensions); 0 = never.  Below
// 1024 dimensions a tile is too few MFMAs for its two barriers and its epilogue.
int wide_min_queries(int nch) {
    if (nch == 24 || nch == 20) return 256;
    if (nch == 16) return 512;
    return 0;
}

static size_t wide_lds_bytes(int nch, int nq) {
    const size_t nq_pad = size_t((nq + kQTile - 1) / kQTile) * kQTile;
    return size_t(kWideRing) * nch * 1024 + nq_pad * 16 + kWideWaves * 32 * 4 + 64;
}

int wide_grid_blocks(int device) {
    hipDeviceProp_t prop;
    int cus = 256;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        cus = prop.multiProcessorCount;
    return cus;      // one 8-wave workgroup per CU: its LDS holds the slice ring
}

template <int NCH, int NB>
static hipError_t launch_wide_n(const ScanArgs &a, int grid, hipStream_t s) {
    const size_t lds = wide_lds_bytes(NCH, a.nq_tile);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_scan_p4_wide<NCH, NB>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((k_scan_p4_wide<NCH, NB>), dim3(grid), dim3(kWideThreads), lds, s, a);
    return hipGetLastError();
}

// a.nq_tile = all queries of the launch (any number up to the chunk size), a.tables = their
// ceil(nq/32) weight tiles back to back, a.qscale / a.qbias / a.gtau indexed by query.
hipError_t launch_scan_p4_wide(const ScanArgs &a, int grid, hipStream_t s) {
    switch (a.nch) {
        case 16: return launch_wide_n<16, 6>(a, grid, s);
        case 20: return launch_wide_n<20, 4>(a, grid, s);
        case 24: return launch_wide_n<24, 2>(a, grid, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace tv
