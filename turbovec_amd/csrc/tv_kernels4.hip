// Scan, score modes L with the u32 or the classic epilogue, append mode, sixteen queries per pass.
//
// The pass of k_scan_lut is bound by LDS reads -- two per code byte and lane, each fetching the
// same table entry of all the launch's queries -- and the LDS serves a wave's 16-byte reads at
// 1.4 times the bytes per clock of its 8-byte ones.  Sixteen queries' tables (16 KiB per chunk of
// 32 byte-groups) do not fit the LDS next to each other for a whole row, so they do not stay: the
// tables of two chunks at a time pass through a double buffer, all 16 waves of the workgroup
// work on the same pair of chunks, and a wave carries the integer sums of its blocks in the
// matrix unit's accumulators from pair to pair until the row is complete.  The tables come
// entry-major (the 16 queries' bytes of an entry side by side) from k_lut_interleave16, so that
// staging them is a plain copy; they are read once per round of 32 blocks per workgroup, from L2.
//
// Sums are taken by v_mfma_i32_16x16x64_i8 against a one-hot B: a lane's looked-up 16 bytes are
// one row of one of the instruction's four k-blocks -- the four lanes r, r + 16, r + 32, r + 48
// look up vector r (or r + 16, in a second accumulator) in the four quarters of a pair of chunks -- and
// B[k][n] = (k % 16 == n) adds byte n of all four into column n: D[r][n] is vector r's sum for
// query n, in the lane that then scores it.  Integers and float epilogues are those of
// turbovec/src/search.rs:1174-1177 (u32) and :516-582 (classic; the definition: :3113-3128),
// term for term.
#include "tv_device.h"
#include "tv_internal.h"

namespace tv {

constexpr int kLut16Threads = 1024;
constexpr int kLut16PairBytes = 2 * 1024 * kLut16Queries;   // two chunks of 1024 entries, 16 bytes each

// dst[tile][chunk][entry][query] = src[tile * 16 + query][chunk][entry]; chunks padded to an even
// number and queries to 16 with zero tables.
__global__ __launch_bounds__(256) void k_lut_interleave16(const uint8_t *src, uint8_t *dst, int nch, int nch_pad, uint32_t nq) {
    const uint32_t e = blockIdx.x * 256 + threadIdx.x;       // (chunk, entry) of the tile
    const uint32_t tile = blockIdx.y;
    const uint32_t cc = e >> 10, ent = e & 1023u;
    if (cc >= uint32_t(nch_pad)) return;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (cc < uint32_t(nch)) {
#pragma unroll
        for (int q = 0; q < kLut16Queries; ++q) {
            const uint32_t qi = tile * kLut16Queries + q;
            if (qi < nq) w[q >> 2] |= uint32_t(src[(size_t(qi) * nch + cc) * 1024 + ent]) << (8 * (q & 3));
        }
    }
    reinterpret_cast<uint4 *>(dst)[(size_t(tile) * nch_pad + cc) * 1024 + ent] = uint4{w[0], w[1], w[2], w[3]};
}

size_t lut16_table_bytes(int nch, size_t nq) {
    const size_t tiles = (nq + kLut16Queries - 1) / kLut16Queries;
    return tiles * size_t((nch + 1) / 2) * kLut16PairBytes;
}

hipError_t launch_lut_interleave16(const uint8_t *d_src, uint8_t *d_dst, int nch, size_t nq, hipStream_t s) {
    const int nch_pad = (nch + 1) / 2 * 2;
    const unsigned tiles = unsigned((nq + kLut16Queries - 1) / kLut16Queries);
    if (tiles == 0) return hipSuccess;
    hipLaunchKernelGGL(k_lut_interleave16, dim3(unsigned(nch_pad) * 4, tiles), dim3(256), 0, s, d_src, d_dst, nch, nch_pad,
                       uint32_t(nq));
    return hipGetLastError();
}

// base + byte E of packed, in one instruction (sub-dword operand select).
template <int E>
__device__ __forceinline__ uint32_t add_byte16(uint32_t base, uint32_t packed) {
    uint32_t r;
    if (E == 0) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 1) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 2) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(base), "v"(packed));
    if (E == 3) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(base), "v"(packed));
    return r;
}

// 16 bytes of LDS per lane, requested behind the compiler's back (it would keep one or two reads in
// flight to save registers, and the wave would sit out every LDS latency); lut_wait<N> on the
// destination holds until at most N younger LDS requests of the wave are outstanding.  Requests of
// other kinds the compiler may have in flight only make that wait longer, never shorter: LDS
// requests complete in order.
template <int OFF>
__device__ __forceinline__ void lut_read16(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
template <int N>
__device__ __forceinline__ void lut_wait(v4i &r) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N) : "memory");
}

// RB = blocks a wave carries through one round of the pairs; kLutAhead = table reads it keeps in
// flight.  CLASSIC: the classic epilogue (search.rs:516-582): the integer sums are flushed into a
// float every 256 byte-groups -- four pairs of chunks -- with fma(scale, f32(sum), fa), fa starting
// at the bias; the score is fa * vec_scale.  (Its sixteen running floats per block take the
// registers of the second block and of two reads in flight.)
template <int RB, bool CLASSIC, int kLutAhead>
__global__ __launch_bounds__(kLut16Threads) void k_scan_lut16(ScanArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    if (launch_switched_off(a.run_if)) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, kb = lane >> 4;
    const int nch = a.nch, npairs = (nch + 1) / 2;
    // blockIdx.y = tile of sixteen queries: a launch may serve several tiles side by side (sampling
    // levels, which leave most of the chip idle one tile at a time); a.nq_tile counts all their queries
    if (blockIdx.y != 0) {
        const size_t ty = blockIdx.y;
        a.tables += ty * size_t(npairs) * kLut16PairBytes;
        a.qscale += ty * kLut16Queries;
        a.qbias += ty * kLut16Queries;
        a.gtau += ty * kQTile;
        a.cand += ty * kLut16Queries * a.seg_stride * kSegCap;
        a.cand_cnt += ty * kLut16Queries * a.seg_stride;
        a.nq_tile -= int(ty) * kLut16Queries;
    }
    if (a.nq_tile > kLut16Queries) a.nq_tile = kLut16Queries;
    uint32_t *scnt = reinterpret_cast<uint32_t *>(smem + 2 * kLut16PairBytes);   // candidates per query of this workgroup
    uint32_t *s_over = scnt + kLut16Queries;                                     // queries whose segment of this workgroup is full
    if (tid < kLut16Queries) scnt[tid] = 0u;
    if (tid == kLut16Queries) *s_over = 0u;

    // the query whose column of the result this lane holds
    const bool qact = r < a.nq_tile;
    const float qs = qact ? a.qscale[r] : 0.0f, qb = qact ? a.qbias[r] : 0.0f;
    const float tau = qact ? order_unkey(a.gtau[r]) : __int_as_float(0x7fc00000);
    v4i bsel = {0, 0, 0, 0};
    bsel[r >> 2] = int(1u << (8 * (r & 3)));

    // table staging: a pair of chunks is 2048 16-byte entries, two per thread
    const uint4 *tsrc = reinterpret_cast<const uint4 *>(a.tables);
    uint4 *tbuf = reinterpret_cast<uint4 *>(smem);
    {
        const uint4 s0 = tsrc[tid], s1 = tsrc[1024 + tid];
        tbuf[tid] = s0;
        tbuf[1024 + tid] = s1;
    }
    const uint32_t lds_base = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem));
    // Which quarter of a pair's lookups this lane makes: chunk ts / 2 of the pair, byte-groups
    // 16 (ts % 2) .. + 15.  A vector's four lanes (r, r + 16, r + 32, r + 48: the four k-blocks of its
    // row) must cover the four quarters, in any order; and the lanes the LDS serves in one cycle of a
    // 16-byte read -- {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same of the upper half (measured:
    // lanes of one such set may read different entries of one 256-byte table at full rate, lanes of two
    // tables with the same bank alignment collide) -- should read the same table: quarters by set.
    const int lp = lane & 31;
    const bool first_set = lp < 4 || (lp >= 12 && lp < 16) || (lp >= 20 && lp < 28);
    const int ts = (lane >> 5) * 2 + (first_set ? 0 : 1);
    // entry (g, sub, v) of a chunk sits at ((g * 2 + sub) * 16 + v) * 16
    const uint32_t lane_off = uint32_t(ts >> 1) * (1024 * kLut16Queries) + uint32_t(ts & 1) * (16 * 512);

    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;
    const uint32_t total_waves = gridDim.x * (kLut16Threads / 64);
    auto live_from = [&](uint32_t j) -> uint32_t {
        if (a.mask == nullptr) return j;
        while (j < nj) {
            const uint32_t b = j * step;
            if (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) != 0u) break;
            j += total_waves;
        }
        return j;
    };
    uint32_t j = live_from(uint32_t(wave) * gridDim.x + blockIdx.x);   // consecutive blocks go to different workgroups
    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes);
    // the 16 bytes this lane looks up for (block b, pair p, vector half): chunk 2 p + ts / 2 (none in
    // the padding chunk of an odd row), byte-groups 16 (ts % 2) .. + 15 of vector r + 16 half
    auto load_codes = [&](uint32_t b, int p, int half) -> uint4 {
        const int c = 2 * p + (ts >> 1);
        if (c >= nch) return uint4{0u, 0u, 0u, 0u};
        return load_stream16(&codes[(size_t(b) * nch + c) * 64 + (ts & 1) * 32 + r + 16 * half]);
    };
    __syncthreads();

    int buf = 0;
    for (;;) {
        uint32_t blk[RB];
        bool has[RB];
        // Once every query's segment of this workgroup is full, every query of the launch is certain
        // to be flagged as overflowed and scanned again from a raised floor: nothing this workgroup
        // could still append would be kept, so it takes no further blocks (rows laid out against the
        // sampler end the launch within a few rounds instead of scoring the whole index for nothing).
        if (*reinterpret_cast<volatile uint32_t *>(s_over) >= uint32_t(a.nq_tile)) j = nj;
#pragma unroll
        for (int i = 0; i < RB; ++i) {
            has[i] = j < nj;
            blk[i] = has[i] ? j * step : 0u;
            if (has[i]) j = live_from(j + total_waves);
        }
        if (!__syncthreads_or(has[0] ? 1 : 0)) break;
        v4i acc[RB][2];
        float fa[RB][2][4];
        uint4 cw[RB][2];
#pragma unroll
        for (int i = 0; i < RB; ++i) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                acc[i][half] = v4i{0, 0, 0, 0};
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) fa[i][half][rr] = qb;
                cw[i][half] = has[i] ? load_codes(blk[i], 0, half) : uint4{0u, 0u, 0u, 0u};
            }
        }
        for (int p = 0; p < npairs; ++p) {
            // the next pair's tables (the first pair's again after the last: the next round's) on their way
            const int pn = p + 1 == npairs ? 0 : p + 1;
            const uint4 s0 = tsrc[size_t(pn) * 2048 + tid], s1 = tsrc[size_t(pn) * 2048 + 1024 + tid];
            uint4 cur[RB][2];
#pragma unroll
            for (int i = 0; i < RB; ++i) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    cur[i][half] = cw[i][half];
                    if (has[i] && p + 1 < npairs) cw[i][half] = load_codes(blk[i], p + 1, half);
                }
            }
            const uint32_t base = lds_base + uint32_t(buf) * kLut16PairBytes + lane_off;
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                if (!has[i]) continue;
                // The block's 64 lookups of this pair as one stream, kLutAhead reads in flight: read n
                // is byte (n / 4) % 16's high (n % 4 < 2) or low nibble entry for vector half n % 2, and
                // goes to that half's accumulator -- consecutive MFMAs alternate between the two chains.
                const uint32_t x0[4] = {cur[i][0].x, cur[i][0].y, cur[i][0].z, cur[i][0].w};
                const uint32_t x1[4] = {cur[i][1].x, cur[i][1].y, cur[i][1].z, cur[i][1].w};
                v4i w[kLutAhead];
                auto issue = [&](auto nn) {
                    constexpr int n = decltype(nn)::value;
                    constexpr int half = n & 1, lo = (n >> 1) & 1, g = n >> 2, d = g >> 2, e = g & 3;
                    const uint32_t xv = half ? x1[d] : x0[d];
                    // nibble * 16 still fits a byte: a mask (and a shift) prepare four entry offsets at once
                    const uint32_t packed = lo ? (xv << 4) & 0xf0f0f0f0u : xv & 0xf0f0f0f0u;
                    lut_read16<g * 512 + lo * 256>(w[n % kLutAhead], add_byte16<e>(base, packed));
                };
                static_for<kLutAhead>(issue);
                static_for<64>([&](auto nn) {
                    constexpr int n = decltype(nn)::value;
                    constexpr int younger = 63 - n < kLutAhead - 1 ? 63 - n : kLutAhead - 1;
                    lut_wait<younger>(w[n % kLutAhead]);
                    if constexpr ((n & 1) == 0) acc[i][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[n % kLutAhead], bsel, acc[i][0], 0, 0, 0);
                    else acc[i][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[n % kLutAhead], bsel, acc[i][1], 0, 0, 0);
                    if constexpr (n + kLutAhead < 64) issue(IntC<n + kLutAhead>{});
                });
            }
            if constexpr (CLASSIC) {
                if ((p & 3) == 3 || p + 1 == npairs) {   // end of a 256-group batch (search.rs:529-531, 577-580)
#pragma unroll
                    for (int i = 0; i < RB; ++i) {
#pragma unroll
                        for (int half = 0; half < 2; ++half) {
#pragma unroll
                            for (int rr = 0; rr < 4; ++rr) fa[i][half][rr] = fmaf(qs, float(uint32_t(acc[i][half][rr])), fa[i][half][rr]);
                            acc[i][half] = v4i{0, 0, 0, 0};
                        }
                    }
                }
            }
            tbuf[(buf ^ 1) * 2048 + tid] = s0;
            tbuf[(buf ^ 1) * 2048 + 1024 + tid] = s1;
            __syncthreads();
            buf ^= 1;
        }
        // D[row][column]: this lane holds rows 4 kb .. + 3 (vectors, + 16 in the second half) of column r
        // (its query): ((f32(acc) * scale) + bias) * vec_scale (search.rs:1174-1177)
#pragma unroll
        for (int i = 0; i < RB; ++i) {
            if (!has[i]) continue;
            const uint32_t b = blk[i];
            uint32_t mw = 0xffffffffu;
            if (a.mask != nullptr) mw = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int v0 = 16 * half + 4 * kb;
                const float4 vs = *reinterpret_cast<const float4 *>(a.scales + size_t(b) * 32 + v0);
                const float vsr[4] = {vs.x, vs.y, vs.z, vs.w};
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const uint32_t slot = b * 32u + uint32_t(v0 + rr);
                    const float s = CLASSIC ? fa[i][half][rr] * vsr[rr] : ((float(acc[i][half][rr]) * qs) + qb) * vsr[rr];
                    if (s >= tau && slot < a.n && ((mw >> (v0 + rr)) & 1u)) {
                        const uint32_t pos = atomicAdd(&scnt[r], 1u);
                        if (pos < kSegCap) a.cand[(size_t(r) * a.seg_stride + blockIdx.x) * kSegCap + pos] = sort_key(s, slot);
                        else if (pos == kSegCap) atomicAdd(s_over, 1u);      // the one append that finds the segment just full
                    }
                }
            }
        }
    }
    __syncthreads();
    if (tid < a.nq_tile) a.cand_cnt[size_t(tid) * a.seg_stride + blockIdx.x] = scnt[tid];
}

constexpr int kLut16RoundBlocks = 2, kLut16RoundBlocksClassic = 1;   // per wave
int lut16_blocks_per_workgroup(bool classic) { return kLut16Threads / 64 * (classic ? kLut16RoundBlocksClassic : kLut16RoundBlocks); }

// One append-mode launch over `tiles` tiles of sixteen queries (the last may hold fewer): a.nq_tile =
// all their queries, a.tables = the first tile's interleaved tables (k_lut_interleave16), floors,
// scales and candidate segments those of the first tile, the others' following at the strides of
// the chunk's layout; a.classic 0 (u32 epilogue) or 1 (classic).
hipError_t launch_scan_lut16(const ScanArgs &a, int grid, int tiles, hipStream_t s) {
    if ((a.classic != 0 && a.classic != 1) || tiles < 1 || a.nq_tile <= (tiles - 1) * kLut16Queries || a.nq_tile > tiles * kLut16Queries)
        return hipErrorInvalidValue;
    const size_t lds = 2 * size_t(kLut16PairBytes) + 128;
    auto launch = [&](auto kernel) -> hipError_t {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(kernel, dim3(grid, tiles), dim3(kLut16Threads), lds, s, a);
        return hipSuccess;
    };
    hipError_t e = a.classic == 1 ? launch(k_scan_lut16<kLut16RoundBlocksClassic, true, 6>) : launch(k_scan_lut16<kLut16RoundBlocks, false, 6>);
    if (e != hipSuccess) return e;
    return hipGetLastError();
}

}  // namespace tv
