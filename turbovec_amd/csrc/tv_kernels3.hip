// Wide batched scan, score mode P, append mode: one pass over the codes serves
// every query of the chunk (up to 1024), not one group of tiles per pass.
//
// A wave decodes its 32-vector block once into registers -- the int8 A operands
// of all its chunks, 8 registers per chunk -- and keeps them there while the
// workgroup walks the query tiles: each tile's weights stream from L2 into LDS
// in slices (half a tile, or a quarter for long rows) through a ring of LDS
// slots, requested four slices ahead by direct-to-LDS loads that use no
// registers; the hand-over of a slice sits in the middle of the previous
// slice's MFMAs.  B operands are read from LDS in one explicitly pipelined
// stream.  The nibble decode and the HBM read of the codes are paid once per
// block instead of once per 96 queries, which leaves the matrix unit as the
// bound: 2 * 32 * 32 * 32 * NCH * 2 int8 operations per (block, tile).
//
// Three shapes of one template: rows of 16 to 24 chunks, one block per wave, 8
// waves per workgroup at 256 registers; rows of 32 to 48 chunks, 4 waves at 512
// registers (A operands partly in AGPRs); rows of 4 to 12 chunks, 2 to 4 blocks
// per wave, every B operand feeding as many MFMAs.
//
// Integers and float epilogue are those of k_scan_p4 (turbovec/src/search.rs:
// 1392-1567, 1519-1524); only the order in which (block, tile) pairs are visited
// differs, and the candidate segments make the result independent of it.  The
// float epilogue is skipped for a tile whose accumulators all stay below an
// integer bound that no passing score can stay below (WideQuery).
#include <algorithm>

#include "tv_device.h"
#include "tv_internal.h"

namespace tv {

constexpr int kWideThreads = 512;    // the widest form (and the matrix-unit probe): 8 waves, 2 per SIMD
constexpr int kWideWaves = kWideThreads / 64;
// LDS slots of one slice each: five when slices are handed over one by one (four requested ahead) or
// two at a time, 2 HO + 1 when more are handed over together.
constexpr int wide_ring(int ho) { return ho <= 2 ? 5 : 2 * ho + 1; }

// 16 bytes per lane from global memory (uniform base + 16 * lane) straight into LDS at
// lds_addr + 16 * lane (lds_addr uniform over the wave).  Counted by the vector-memory counter
// like a load.  Uniform bases live in scalar registers: the kernel has no vector register to spare.
__device__ __forceinline__ void dma16_to_lds(uint32_t lds_addr, const void *sbase, uint32_t lane16) {
    const uint32_t u = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_addr)));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(u), "v"(lane16), "s"(sbase) : "memory", "m0");
}

// 16 bytes per lane from uniform base + 16 * lane into registers, invisible to the compiler's
// wait-count bookkeeping (wait_vm<N> on the destination is the matching wait).
__device__ __forceinline__ void load16_async_s(u32x4 &dst, const void *sbase, uint32_t lane16) {
    asm volatile("global_load_dwordx4 %0, %1, %2 nt" : "=&v"(dst) : "v"(lane16), "s"(sbase));
}

// One word of LDS by its address, read afresh every time.
__device__ __forceinline__ uint32_t lds_word(uint32_t addr) {
    return *reinterpret_cast<const volatile __attribute__((address_space(3))) uint32_t *>(uintptr_t(addr));
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

// The int8 MFMA as hand-written instructions, for the forms of the kernel whose A operands do not
// all fit the vector registers: an operand the compiler keeps in an accumulation register is copied
// to a vector register before every use (four moves per MFMA, on the one wave of the SIMD that also
// has to issue the MFMAs), while the instruction itself can read it where it is.  ACC_REG picks
// the register file of the A operand; the accumulator stays in vector registers.  The compiler does
// not know these are matrix instructions: the wait before their result is read is written out
// (mfma_settle), and a tile's first MFMA takes the constant zero as its addend.
template <bool ACC_REG>
__device__ __forceinline__ void mfma_i8_first(v16i &acc, const v4i &a, const v4i &b) {
    if constexpr (ACC_REG) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0" : "=&v"(acc) : "a"(a), "v"(b));
    else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
}
template <bool ACC_REG>
__device__ __forceinline__ void mfma_i8_add(v16i &acc, const v4i &a, const v4i &b) {
    if constexpr (ACC_REG) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "a"(a), "v"(b));
    else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
// An 8-pass MFMA's result may be read by the vector ALU 11 wait states after the instruction at
// the earliest; 20 are spent.
__device__ __forceinline__ void mfma_settle(v16i &acc) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc)); }

// Per query, in LDS.  A score is fmaf(float(acc), qs, qb) * row_scale and passes when it reaches
// tau.  With tau, qs > 0 and row scales >= 0 that needs acc >= (tau / max_row_scale - qb) / qs, up
// to rounding: ta / max_row_scale - tb is that bound in accumulator units with the roundings of
// both sides priced in (relative 1e-5, against a few 2^-24, plus 2 for the integer conversions),
// so comparing the largest accumulator of a lane with it never loses a candidate and lets the
// common tile -- no candidate at all -- skip the float epilogue.
// 24 bytes per query, in two arrays: what every tile reads (the bound, with the query's scale and
// bias beside it for the rare float score), and what only an append touches.
struct WideQuery {
    float ta, tb;           // ta = -inf: no such bound, always score (tau <= 0, open floor, odd qs); +inf: padding query
};
struct WideQueryTail {
    float qs, qb, tau;      // tau is NaN for the padding queries of the last tile: nothing passes
    uint32_t cnt;           // candidates this workgroup appended
};
constexpr int kWideQueryBytes = int(sizeof(WideQuery) + sizeof(WideQueryTail));
constexpr int kWideTableBytes = 1024;    // the byte table of the split decode (kDecodeBytes), padded to the ring's alignment

// WAVES = 8 (two per SIMD, 256 VGPRs each) holds rows of up to 24 chunks; WAVES = 4 (one per SIMD)
// gives a wave the whole 512-register file -- the compiler keeps what does not fit the VGPRs in
// AGPRs -- for rows of up to 48 chunks.  A tile's weights go through the ring in SPT slices of
// NCH / SPT chunks, handed over one by one (HO = 1) or HO at a time.  Short rows leave registers
// for BLK blocks per wave: every B operand read from LDS then feeds BLK MFMAs, and a tile's
// barriers and epilogue are shared by BLK times the work.
//
// KS = 2 splits a row of 2 * NCH chunks over a pair of waves (w, w + 1): each holds the block's
// operands for half the row (NCH chunks: what one wave's registers take), walks its half of every
// tile's weights -- a ring slot then carries both halves of a slice side by side -- and at the
// end of a tile the odd wave hands its partial sums to the even one through LDS, which adds them
// and does the tile's bound test and scoring.  Two blocks per workgroup instead of four, one more
// barrier per tile: the form for rows beyond what one wave holds.
//
// SPLIT: the block phase decodes half of every chunk through the byte table in LDS, like
// k_scan_p4 (code bytes 0-7 of a lane on the vector ALU, bytes 8-15 looked up whole); the weights
// then come in that kernel's split order.  The decode is the block phase -- both waves of a SIMD
// at it together, the matrix unit idle -- and the LDS has nothing else to do then.
template <int NCH, int NB, int WAVES, int SPT, int BLK, int HO, int KS, bool SPLIT = false>
__global__ __launch_bounds__(WAVES * 64, WAVES == 8 ? 2 : 1) void k_scan_p4_wide(ScanArgs a) {
    static_assert(NCH % SPT == 0, "a slice is a whole number of chunks");
    static_assert(!SPLIT || (WAVES == 8 && BLK == 1 && KS == 1), "the split decode is built for the one-block eight-wave forms");
    static_assert(KS == 1 || (KS == 2 && WAVES == 4 && BLK == 1 && HO == 1), "row halves go to the wave pairs of the four-wave form");
    constexpr int kWideRing = wide_ring(HO);
    static_assert(HO == 1 || (SPT % HO == 0 && kWideRing >= 2 * HO + 1), "slices handed over together must fit the ring twice");
    extern __shared__ __align__(16) uint8_t smem_all[];
    if (launch_switched_off(a.run_if)) return;
    // (the byte table, when there is one, sits at the start of the kernel's LDS -- no static
    // allocation precedes it -- so that a code byte's offset in it is its address)
    // (... and the slice ring behind it keeps the 1 KiB alignment of its direct-to-LDS loads)
    uint8_t *smem = smem_all + (SPLIT ? kWideTableBytes : 0);
    constexpr int kWideThreads = WAVES * 64, kWideWaves = WAVES;
    constexpr int kSC = NCH / SPT;                          // chunks per slice
    constexpr int kM = 2 * kSC;                             // MFMAs per wave and slice: (low, high) of each chunk
    constexpr int kSlice = kM * 1024;                       // bytes: one 1 KiB B operand per MFMA
    constexpr int kSlot = KS * kSlice;                      // a ring slot: the slice of every row part
    constexpr int kLoaders = kWideWaves / KS;               // waves that share the loading of one row part's slice
    constexpr int kPieces = kM / kLoaders;                  // direct-to-LDS loads per wave and slice ...
    constexpr int kExtra = kM % kLoaders;                   // ... plus one more in the first kExtra waves
    static_assert(KS == 1 || kExtra == 0, "the pair form deals a slice's pieces evenly");
    constexpr int kAhead = kWideRing - 1;
    // Four-wave forms (one wave per SIMD, up to 48 chunks = 384 operand registers): chunks from
    // kVecChunks on live in accumulation registers and the MFMAs are written by hand.
    constexpr bool kHandMfma = WAVES == 4 && BLK == 1;
    constexpr int kVecChunks = 22;
    static_assert(!kHandMfma || (NCH - kVecChunks) * 8 <= 256, "operands beyond the vector registers must fit the accumulation registers");
    const int nq = a.nq_tile;
    const int nt = (nq + kQTile - 1) / kQTile;
    const int nq_pad = nt * kQTile;
    const int n_slices = SPT * nt;                          // per pass over the tiles; the host guarantees >= kAhead
    WideQuery *sq = reinterpret_cast<WideQuery *>(smem + kWideRing * kSlot);
    WideQueryTail *sqt = reinterpret_cast<WideQueryTail *>(sq + nq_pad);
    float *s_vs = reinterpret_cast<float *>(sqt + nq_pad);  // [waves][BLK][32]: row scales, NaN where not allowed
    uint32_t *snext = reinterpret_cast<uint32_t *>(s_vs + kWideWaves * BLK * 32);
    v4i *s_xch = reinterpret_cast<v4i *>(snext + 16);       // KS = 2: [pairs][4][64 lanes] partial sums on their way
    const uint32_t lds_b = uint32_t(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) uint8_t *)smem));

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int qn = lane & 31, h = lane >> 5;
    const uint32_t lane16 = uint32_t(lane) * 16;
    const int part = KS == 2 ? (wave & 1) : 0;              // which half of the row this wave holds
    const int loader = KS == 2 ? (wave >> 1) : wave;        // its rank among the waves loading that part's slices
    for (int q = tid; q < nq_pad; q += kWideThreads) {
        const bool act = q < nq;
        const float qs = act ? a.qscale[q] : 0.0f, qb = act ? a.qbias[q] : 0.0f;
        const float tau = act ? order_unkey(a.gtau[q]) : __int_as_float(0x7fc00000);
        sqt[q].qs = qs;
        sqt[q].qb = qb;
        sqt[q].tau = tau;
        sqt[q].cnt = 0u;
        const float inf = __int_as_float(0x7f800000);
        // The bound's error analysis assumes normal floats throughout: outside 1e-30 .. 1e30
        // (subnormal floors round coarsely; tau / qs may overflow and still be met by a huge row
        // scale) there is no bound and every tile is scored.
        const bool bounded = tau >= 1e-30f && tau <= 1e30f && qs >= 1e-30f && qs <= 1e30f && fabsf(qb) <= 1e30f &&
                             tau / qs < inf;
        const float rb = qb / qs;
        sq[q].ta = !act ? inf : bounded ? (tau / qs) * (1.0f - 1e-5f) : -inf;
        sq[q].tb = act && bounded ? rb + 1e-5f * fabsf(rb) + 2.0f : 0.0f;
    }
    if constexpr (SPLIT) {
        for (int b = tid; b < 256; b += kWideThreads) {
            const uint32_t lo = (a.lv[(b & 15) >> 2] >> (8 * (b & 3))) & 0xffu;
            const uint32_t hi = (a.lv[b >> 6] >> (8 * ((b >> 4) & 3))) & 0xffu;
            reinterpret_cast<uint16_t *>(smem_all)[b] = uint16_t(lo | (hi << 8));
        }
    }
    if (tid == 0) { snext[0] = 0u; snext[1] = 0u; snext[2] = 0u; snext[3] = 0u; snext[4] = 0u; }
    uint32_t *s_over = snext + 1;                           // queries whose segment of this workgroup is full
    const uint32_t s_over_addr = lds_b + uint32_t(reinterpret_cast<uint8_t *>(s_over) - smem);
    __syncthreads();

    const uint32_t t0 = a.lv[0], t1 = a.lv[1], t2 = a.lv[2], t3 = a.lv[3];
    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;

    // next live block of this workgroup (blocks m * gridDim.x + blockIdx.x), claimed wave by wave;
    // the two waves of a pair must arrive at the same block without talking: pair p takes the
    // logical blocks m = p, p + pairs, ...
    uint32_t pair_m = uint32_t(wave >> 1);
    auto claim = [&]() -> uint32_t {
        for (;;) {
            uint32_t m = 0;
            if constexpr (KS == 2) {
                m = pair_m;
                pair_m += kWideWaves / 2;
            } else {
                if (lane == 0) m = atomicAdd(snext, 1u);
                m = uint32_t(__builtin_amdgcn_readfirstlane(int(m)));
            }
            const uint32_t j = m * gridDim.x + blockIdx.x;
            if (j >= nj || a.mask == nullptr) return j;
            const uint32_t b = j * step;
            if (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) != 0u) return j;
        }
    };

    // The weights are one periodic stream of slices (slice s = part s % SPT of tile s / SPT, kSlice
    // contiguous bytes; after the last tile the first follows again for the next round of blocks).
    // Stream position g lives in ring slot g % kWideRing.  Half way through the MFMAs of slice g
    // every wave waits for its own pieces of slice g + 1, meets the others at a barrier -- after
    // which slice g + 1 is whole and slice g - 1 is read by nobody -- and requests slice g + 4 into
    // the slot of g - 1.  The hand-over thus sits inside a run of MFMAs, where the SIMD's other wave
    // keeps the matrix unit busy, and a wave that finishes slice g starts g + 1 without waiting.
    // At that wait the requests for slices g + 2 and g + 3 are younger: 2 * pieces stay outstanding
    // (waves below kExtra request one piece more).
    int req_slice = 0, req_slot = 0;                        // next stream position to request
    auto request_next = [&]() {
        // KS = 1: the stream is contiguous in memory.  KS = 2: a tile holds the first half of the
        // row's chunks, then the second; slice s is part s % SPT of each half of tile s / SPT.
        const uint8_t *src = KS == 1 ? a.tables + size_t(req_slice) * kSlice + size_t(loader) * 1024
                                     : a.tables + size_t(req_slice / SPT) * (size_t(KS) * NCH * 2048) +
                                           size_t(part) * (NCH * 2048) + size_t(req_slice % SPT) * kSlice + size_t(loader) * 1024;
        const uint32_t dst = lds_b + uint32_t(req_slot) * kSlot + uint32_t(part) * kSlice + uint32_t(loader) * 1024;
#pragma unroll
        for (int p = 0; p < kPieces; ++p)
            dma16_to_lds(dst + uint32_t(p) * (kLoaders * 1024), src + size_t(p) * (kLoaders * 1024), lane16);
        if (kExtra != 0 && wave < kExtra)
            dma16_to_lds(dst + uint32_t(kPieces) * (kLoaders * 1024), src + size_t(kPieces) * (kLoaders * 1024), lane16);
        req_slice = req_slice + 1 == n_slices ? 0 : req_slice + 1;
        req_slot = req_slot + 1 == kWideRing ? 0 : req_slot + 1;
    };
    auto hand_over = [&](auto younger_slices) {
        constexpr int ys = decltype(younger_slices)::value;
        if (kExtra != 0 && wave < kExtra)
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(ys * (kPieces + 1)) : "memory");
        else
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(ys * kPieces) : "memory");
        __syncthreads();
        request_next();
    };
    // HO > 1: one hand-over per HO slices, in the middle of the last of them.  By then every wave
    // is past slices g - HO .. g - 1 (g = the slice in progress); each wave's pieces of the HO
    // slices after g, requested at the hand-over before, must have landed (nothing younger is in
    // flight: the wait is for everything); after the barrier those are whole and the HO slices
    // behind g are free: the next HO slices are requested into their slots.
    auto hand_over_group = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int i = 0; i < HO; ++i) request_next();
    };
    if constexpr (HO == 1) {
        // slices 0..3 requested, slice 0 whole: the state the first hand-over expects
        for (int i = 0; i < kAhead - 1; ++i) request_next();
        hand_over(IntC<kAhead - 2>{});
    } else {
        // slices 0 .. 2 HO - 1 requested and whole: the state the first group hand-over expects
        for (int i = 0; i < 2 * HO; ++i) request_next();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
    int use_slot = 0;                                       // ring slot of the slice consumed next

    v4i alo[BLK][NCH], ahi[BLK][NCH];
    v16i acc[BLK];
    // B operands travel through NB registers requested NB MFMAs ahead, in one stream that runs on
    // from a slice into the next (whole since the hand-over in the middle of the current one): a
    // wave opens the stream at the start of a round of tiles and closes it at the end.
    static_assert(kM % NB == 0 && NB <= kM / 2, "the operand ring must line up with the slices");
    v4i w[NB];
    auto open_stream = [&]() {
        const uint32_t baddr = lds_b + uint32_t(use_slot) * kSlot + uint32_t(part) * kSlice + lane16;
        static_for<NB>([&](auto mm) { lds_read16_async<decltype(mm)::value * 1024>(w[decltype(mm)::value], baddr); });
    };
    auto close_stream = [&]() {    // the reads into the slice after the round's last are dropped, once landed
        static_for<NB>([&](auto mm) { lds_wait<0>(w[decltype(mm)::value]); });
    };
    // The kM MFMAs of one slice.  MFMA m takes chunk PART * kSC + m/2 (low nibbles for even m,
    // high for odd) against the 1 KiB of weights at m * 1024; the hand-over of the next slice
    // sits in the middle.
    auto slice_mfmas = [&](auto slice_no) {
        constexpr int c0 = decltype(slice_no)::value * kSC;
        const uint32_t baddr = lds_b + uint32_t(use_slot) * kSlot + uint32_t(part) * kSlice + lane16;
        use_slot = use_slot + 1 == kWideRing ? 0 : use_slot + 1;
        const uint32_t naddr = lds_b + uint32_t(use_slot) * kSlot + uint32_t(part) * kSlice + lane16;
        static_for<kM>([&](auto mm) {
            constexpr int m = decltype(mm)::value;
            if constexpr (m == kM / 2) {
                if constexpr (HO == 1) hand_over(IntC<kAhead - 2>{});
                else if constexpr (decltype(slice_no)::value % HO == HO - 1) hand_over_group();
            }
            lds_wait<NB - 1>(w[m % NB]);
            static_for<BLK>([&](auto kk) {
                constexpr int k = decltype(kk)::value;
                constexpr int c = c0 + m / 2;
                if constexpr (kHandMfma) {
                    const v4i &A = (m & 1) == 0 ? alo[k][c] : ahi[k][c];
                    if constexpr (decltype(slice_no)::value == 0 && m == 0) mfma_i8_first<(c >= kVecChunks)>(acc[k], A, w[m % NB]);
                    else mfma_i8_add<(c >= kVecChunks)>(acc[k], A, w[m % NB]);
                } else if constexpr ((m & 1) == 0) {
                    acc[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo[k][c], w[m % NB], acc[k], 0, 0, 0);
                } else {
                    acc[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi[k][c], w[m % NB], acc[k], 0, 0, 0);
                }
            });
            if constexpr (m + NB < kM) lds_read16_async<(m + NB) * 1024>(w[m % NB], baddr);
            else lds_read16_async<(m + NB - kM) * 1024>(w[m % NB], naddr);
        });
    };

    int inv_vmax[BLK];       // bits of 1 / (largest allowed row scale of the block); +inf when that is 0
    bool odd_block[BLK];
    uint32_t blk[BLK];       // the wave's blocks of this round
    uint32_t round_no = 0;
    for (;;) {
        // ---- block phase: claim, load, decode into registers ----
        bool has = false;
        // Once every query's segment of this workgroup is full, every query of the launch is
        // certain to be flagged as overflowed and scanned again from a raised floor: nothing this
        // workgroup could still append would be kept, so it claims no further blocks.  (A floor
        // far too low -- rows arranged against the sampler -- ends the launch within a few rounds
        // instead of scoring the whole index for nothing.)
        // (The two waves of a pair must see the same value -- one claiming a block while its partner
        // sits out would add stale partial sums -- so the pair form reads it behind a barrier every
        // wave's appends of the round before have passed.)
        if constexpr (KS == 2) __syncthreads();
        // (read as LDS, not through a generic pointer: a flat load is counted by both memory
        // counters and the compiler would wait for every weight request in flight before it)
        const bool futile = uint32_t(__builtin_amdgcn_readfirstlane(int(lds_word(s_over_addr)))) >= uint32_t(nq);
        static_for<BLK>([&](auto kk) {
            constexpr int k = decltype(kk)::value;
            const uint32_t j = futile ? nj : claim();
            const bool has_k = j < nj;
            has = has || has_k;
            const uint32_t b = has_k ? j * step : 0u;
            blk[k] = b;
            float sc = __int_as_float(0x7fc00000);
            bool ok = false;
            if (has_k) {
                // the whole block in one burst: the previous block's operands are dead by now, so
                // the raw codes (4 VGPRs per chunk) and the operands decoded from them so far (8 per
                // chunk) fit the registers the operands alone need at the end
                const uint8_t *p = a.codes + (size_t(b) * KS + size_t(part)) * (NCH * 1024);
                u32x4 raw[NCH];
                // with hand-written MFMAs the chunks bound for the accumulation registers come
                // first: their raw codes leave the vector registers before the others' operands grow
                constexpr int kFirst = kHandMfma && NCH > kVecChunks ? kVecChunks : 0;
                static_for<NCH>([&](auto ii) {
                    constexpr int c = (decltype(ii)::value + kFirst) % NCH;
                    load16_async_s(raw[c], p + size_t(c) * 1024, lane16);
                });
                uint32_t te[2][4], to[2][4];    // (split decode) table entries on their way, this chunk's and the next's
                static_for<NCH>([&](auto ii) {
                    constexpr int c = (decltype(ii)::value + kFirst) % NCH;
                    wait_vm<NCH - 1 - decltype(ii)::value>(raw[c]);
                    const uint32_t x[4] = {raw[c].x, raw[c].y, raw[c].z, raw[c].w};
                    if constexpr (SPLIT) {
                        // the chunk's first operand from code bytes 0..7 on the vector ALU (low-nibble
                        // levels of bytes 0..3, high-nibble levels of bytes 0..3, the same of 4..7), the
                        // second from bytes 8..15 through the table: dword r = entries of bytes 8+2r
                        // and 9+2r.  The next chunk's entries are requested before this chunk's are
                        // waited for, so that the LDS answers while the ALU works.  No other LDS or
                        // scalar-memory request of this wave is in flight here (the B stream is
                        // closed, the claim has returned), so the counts are exact.
                        constexpr int i = decltype(ii)::value, p = i & 1;
                        auto request = [&](auto cc, auto pp) {
                            constexpr int cn = decltype(cc)::value, pn = decltype(pp)::value;
                            const uint32_t xa = raw[cn].z, xb = raw[cn].w;
                            lds_u16(te[pn][0], byte_x2<0>(xa)); lds_u16(to[pn][0], byte_x2<1>(xa));
                            lds_u16(te[pn][1], byte_x2<2>(xa)); lds_u16(to[pn][1], byte_x2<3>(xa));
                            lds_u16(te[pn][2], byte_x2<0>(xb)); lds_u16(to[pn][2], byte_x2<1>(xb));
                            lds_u16(te[pn][3], byte_x2<2>(xb)); lds_u16(to[pn][3], byte_x2<3>(xb));
                        };
                        if constexpr (i == 0) request(IntC<c>{}, IntC<p>{});
                        if constexpr (i + 1 < NCH) {
                            constexpr int cn = (i + 1 + kFirst) % NCH;
                            wait_vm<NCH - 2 - i>(raw[cn]);
                            request(IntC<cn>{}, IntC<1 - p>{});
                        }
                        alo[k][c][0] = int(levels_of(x[0] & 0x0f0f0f0fu, t0, t1, t2, t3));
                        alo[k][c][1] = int(levels_of((x[0] >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3));
                        alo[k][c][2] = int(levels_of(x[1] & 0x0f0f0f0fu, t0, t1, t2, t3));
                        alo[k][c][3] = int(levels_of((x[1] >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3));
                        if constexpr (i + 1 < NCH)
                            asm volatile("s_waitcnt lgkmcnt(8)"
                                         : "+v"(te[p][0]), "+v"(te[p][1]), "+v"(te[p][2]), "+v"(te[p][3]), "+v"(to[p][0]), "+v"(to[p][1]), "+v"(to[p][2]), "+v"(to[p][3])
                                         :: "memory");
                        else
                            asm volatile("s_waitcnt lgkmcnt(0)"
                                         : "+v"(te[p][0]), "+v"(te[p][1]), "+v"(te[p][2]), "+v"(te[p][3]), "+v"(to[p][0]), "+v"(to[p][1]), "+v"(to[p][2]), "+v"(to[p][3])
                                         :: "memory");
#pragma unroll
                        for (int d = 0; d < 4; ++d) ahi[k][c][d] = int(te[p][d] | (to[p][d] << 16));
                        // one chunk after the other: left to itself the scheduler works on several at
                        // once and runs out of registers
                        asm volatile("" : "+v"(alo[k][c]), "+v"(ahi[k][c]));
                    } else {
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            alo[k][c][d] = int(levels_of(x[d] & 0x0f0f0f0fu, t0, t1, t2, t3));
                            ahi[k][c][d] = int(levels_of((x[d] >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3));
                        }
                    }
                    if constexpr (kHandMfma && c >= kVecChunks) {
                        // into its accumulation registers now, not at the first MFMA that reads it
                        asm volatile("" : "+a"(alo[k][c]));
                        asm volatile("" : "+a"(ahi[k][c]));
                    }
                });
                const uint32_t slot = b * 32u + uint32_t(lane & 31);
                ok = slot < a.n;
                if (ok && a.mask != nullptr) ok = (uint32_t(a.mask[b >> 1] >> ((b & 1) * 32)) >> (lane & 31)) & 1u;
                if (ok) sc = a.scales[slot];
            }
            // row scales (NaN where not allowed, and for a block slot left empty: its stale
            // operands then score nothing); their maximum over the allowed rows feeds the
            // accumulator bound, and a block with a negative, huge or non-finite one (no encoder
            // writes such) is always scored
            if (lane < 32) s_vs[(wave * BLK + k) * 32 + lane] = sc;
            float vmax = ok ? sc : 0.0f;
            const bool odd = ok && !(sc >= 0.0f && sc <= 1e30f);
#pragma unroll
            for (int d = 16; d >= 1; d >>= 1) vmax = fmaxf(vmax, __shfl_xor(vmax, d));
            // A largest row scale below 1e-30 (a foreign snapshot may hold subnormal scales; no
            // encoder writes them) has a reciprocal that overflows or rounds coarsely: such a
            // block is always scored too.  All scales zero: every score is zero, below any
            // positive floor, and the infinite bound is right.
            const float inv = 1.0f / vmax;
            odd_block[k] = __any(odd) || (vmax > 0.0f && vmax < 1e-30f);
            inv_vmax[k] = __builtin_amdgcn_readfirstlane(__float_as_int(inv));
        });
        if constexpr (SPLIT) {
            // "does any wave have a block?" through three rotating LDS flags instead of
            // __syncthreads_or, whose static LDS word would sit in front of the byte table: round r
            // sets and reads flag r % 3 on either side of the barrier and clears the next round's,
            // which every wave has finished reading (two barriers ago).
            uint32_t *flag = snext + 2;
            if (tid == 0) flag[(round_no + 1) % 3u] = 0u;
            if (has && lane == 0) flag[round_no % 3u] = 1u;
            __syncthreads();
            const bool any = __builtin_amdgcn_readfirstlane(int(lds_word(s_over_addr + 4u + 4u * (round_no % 3u)))) != 0;   // (uniform, and known to be)
            ++round_no;
            if (!any) break;
        } else {
            if (!__syncthreads_or(has ? 1 : 0)) break;
        }

        // ---- tile phase ----
        // Scores of tile t for block k of this wave; lane owns query t*32 + qn and rows
        // 8*(r/4) + 4*h + r%4 (search.rs:1519-1524).  Entered only when some lane's largest
        // accumulator reaches its query's bound, and then only the accumulators that reach it
        // (one or two in the whole wave, as a rule) are scored and, if they pass, appended.
        auto score_tile = [&](int q, int bound, auto kk) {
            constexpr int k = decltype(kk)::value;
            const float4 qp = *reinterpret_cast<const float4 *>(&sqt[q].qs);
            const float qs = qp.x, qb = qp.y, tau = qp.z;
            const float *vs = s_vs + (wave * BLK + k) * 32 + 4 * h;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                if (acc[k][r] >= bound) {
                    const int i = 8 * (r >> 2) + (r & 3);
                    const float s = fmaf(float(acc[k][r]), qs, qb) * vs[i];
                    if (s >= tau) {
                        const uint32_t pos = atomicAdd(&sqt[q].cnt, 1u);
                        if (pos < kSegCap)
                            a.cand[(size_t(q) * a.seg_stride + blockIdx.x) * kSegCap + pos] =
                                sort_key(s, blk[k] * 32u + uint32_t(i + 4 * h));
                        else if (pos == kSegCap)
                            atomicAdd(s_over, 1u);      // the one append that finds the segment just full
                    }
                }
            }
        };
        // A first sampling level without floors (a.best_of_block): per tile and block the lane's best
        // allowed row, the better of the two lanes that share a query, one candidate per block and
        // query -- a real score of a real row, so the k-th best of these is a floor k scanned rows
        // reach.  One launch over a round of blocks; the hot loop never comes here.
        auto best_tile = [&](int q, auto kk) {
            constexpr int k = decltype(kk)::value;
            const float2 qp = *reinterpret_cast<const float2 *>(&sqt[q].qs);
            const float qs = qp.x, qb = qp.y;
            const float *vs = s_vs + (wave * BLK + k) * 32 + 4 * h;
            float bs = 0.0f;
            int bi = -1;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = 8 * (r >> 2) + (r & 3);
                const float s = fmaf(float(acc[k][r]), qs, qb) * vs[i];
                if (s == s && (bi < 0 || s > bs)) { bs = s; bi = i + 4 * h; }    // rows in rising order: ties keep the lower slot
            }
            const float os_ = __shfl_xor(bs, 32);
            const int oi = __shfl_xor(bi, 32);
            if (oi >= 0 && (bi < 0 || os_ > bs || (os_ == bs && oi < bi))) { bs = os_; bi = oi; }
            if (h == 0 && bi >= 0 && q < nq) {
                const uint32_t pos = atomicAdd(&sqt[q].cnt, 1u);
                if (pos < kSegCap)
                    a.cand[(size_t(q) * a.seg_stride + blockIdx.x) * kSegCap + pos] = sort_key(bs, blk[k] * 32u + uint32_t(bi));
            }
        };
        const bool best_mode = BLK == 1 && a.best_of_block != 0;   // (several blocks per wave: no registers to spare for it)
        if (has) open_stream();
        for (int t = 0; t < nt; ++t) {
            const int q = t * kQTile + qn;
            if (has) {
                if constexpr (!kHandMfma)
                    static_for<BLK>([&](auto kk) { acc[decltype(kk)::value] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; });
                slice_mfmas(IntC<0>{});
                // the tile's accumulator bounds, fetched and converted under the MFMAs
                const float2 tq = *reinterpret_cast<const float2 *>(&sq[q].ta);
                int bound[BLK];
                static_for<BLK>([&](auto kk) {
                    constexpr int k = decltype(kk)::value;
                    const float bf = fmaf(tq.x, __int_as_float(inv_vmax[k]), -tq.y) - 1.0f;
                    asm("v_cvt_i32_f32 %0, %1" : "=v"(bound[k]) : "v"(bf));   // saturates; NaN gives 0
                    if (odd_block[k]) bound[k] = int(0x80000000);
                });
                static_for<SPT - 1>([&](auto pp) { slice_mfmas(IntC<decltype(pp)::value + 1>{}); });
                if constexpr (KS == 2) {
                    // the odd wave's half of the sums crosses to the even one; the slot is free
                    // again by the time it is written next: a hand-over barrier lies in between
                    mfma_settle(acc[0]);
                    v4i *x = s_xch + (wave >> 1) * 256 + lane;
                    if (part == 1) {
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4)
                            x[r4 * 64] = v4i{acc[0][4 * r4], acc[0][4 * r4 + 1], acc[0][4 * r4 + 2], acc[0][4 * r4 + 3]};
                    }
                    __syncthreads();
                    if (part == 0) {
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4) {
                            const v4i o = x[r4 * 64];
                            acc[0][4 * r4] += o[0]; acc[0][4 * r4 + 1] += o[1]; acc[0][4 * r4 + 2] += o[2]; acc[0][4 * r4 + 3] += o[3];
                        }
                    }
                }
                if (KS == 1 || part == 0) static_for<BLK>([&](auto kk) {
                    constexpr int k = decltype(kk)::value;
                    if constexpr (kHandMfma && KS == 1) mfma_settle(acc[k]);
                    if constexpr (BLK == 1) {
                        if (best_mode) { best_tile(q, kk); return; }
                    }
                    const v16i &c = acc[k];
                    int m0 = max(max(c[0], c[1]), c[2]), m1 = max(max(c[3], c[4]), c[5]);
                    int m2 = max(max(c[6], c[7]), c[8]), m3 = max(max(c[9], c[10]), c[11]);
                    m0 = max(max(m0, c[12]), c[13]);
                    m1 = max(max(m1, c[14]), c[15]);
                    if (max(max(m0, m1), max(m2, m3)) >= bound[k]) score_tile(q, bound[k], kk);
                });
            } else {
                use_slot = (use_slot + SPT) % kWideRing;
                if constexpr (HO == 1) {
#pragma unroll
                    for (int i = 0; i < SPT; ++i) hand_over(IntC<kAhead - 2>{});
                } else {
#pragma unroll
                    for (int i = 0; i < SPT / HO; ++i) hand_over_group();
                }
                if constexpr (KS == 2) __syncthreads();     // the tile's exchange barrier, met by every wave
            }
        }
        if (has) close_stream();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // requests still in flight write this workgroup's LDS
    __syncthreads();
    for (int q = tid; q < nq; q += kWideThreads) a.cand_cnt[size_t(q) * a.seg_stride + blockIdx.x] = sqt[q].cnt;
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

// Smallest chunk of queries the wide kernel is the faster one for; 0 = no instance for this row
// length.  Measured against the tile-group kernels on 4-bit indexes of 256 to 3072 dimensions:
// the wide kernel wins as soon as the tile-group kernel would need a second pass over the codes
// (it serves 128 queries per pass up to 1024 dimensions, 96 at 1280 and 1536), by 1.4 to 1.6
// times at 1024 queries; at 1792 to 2304 dimensions, where two tiles' weights stay resident, it is
// level at 97 to 128 queries (two tile-group passes); from 2560 dimensions the tile-group kernel
// streams four tiles' weights and serves 128 queries in one pass, 1 to 7 % faster than the wide
// kernel there, which takes over from 129 (1.2 to 1.4 times faster at 160 to 384 queries, 1.6 to
// 1.7 times at 1024).
int wide_min_queries(int nch) {
    switch (nch) {
        case 2: case 4: case 6: case 8: case 10: case 12: case 14: case 16: case 18: return 129;
        case 20: case 22: case 24: return 97;
        case 28: case 32: case 36: return 97;
        case 40: case 44: case 48: return 129;
        case 56: case 64: case 72: case 80: case 88: case 96: return 129;
        default: return 0;
    }
}

// Whether the instance for this row length serves a first level without floors (ScanArgs::best_of_block).
bool wide_serves_best_of_block(int nch) { return nch >= 12 && wide_blocks_per_workgroup(nch) > 0; }

// Blocks one workgroup of the instance for this row length holds per round (waves x blocks per
// wave, or wave pairs); 0 = no instance.
int wide_blocks_per_workgroup(int nch) {
    switch (nch) {
        case 2: return 48;
        case 4: return 32;
        case 6: return 24;
        case 8: case 10: return 16;
        case 12: case 14: case 16: case 18: case 20: case 22: case 24: return 8;
        case 28: case 32: case 36: case 40: case 44: case 48: return 4;
        case 56: case 64: case 72: case 80: case 88: case 96: return 2;
        default: return 0;
    }
}

static size_t wide_lds_bytes(int ring, int slot_bytes, int nq, int blk, int ks, bool split = false) {
    const size_t nq_pad = size_t((nq + kQTile - 1) / kQTile) * kQTile;
    return size_t(ring) * slot_bytes + nq_pad * kWideQueryBytes + size_t(kWideWaves) * blk * 32 * 4 + 64 +
           (ks == 2 ? 2 * 4096 : 0) + (split ? kWideTableBytes : 0);
}

// Most queries (whole tiles) a launch with this ring fits into the 160 KiB of LDS.
static int wide_max_queries_of(int ring, int slot_bytes, int blk, int ks, bool split = false) {
    const size_t fixed = wide_lds_bytes(ring, slot_bytes, 0, blk, ks, split);
    if (fixed >= 160 * 1024) return 0;
    return int((160 * 1024 - fixed) / kWideQueryBytes / kQTile * kQTile);
}

// Most queries one launch of the instance(s) for this row length serves (0: no instance); at least
// 1024 wherever there is one.
int wide_max_queries(int nch) {
    switch (nch) {
        case 24: return std::min(2048, wide_max_queries_of(wide_ring(4), 12 * 1024, 1, 1, wide_weights_split(24)));
        default: return wide_blocks_per_workgroup(nch) > 0 ? 1024 : 0;
    }
}

int wide_grid_blocks(int device) {
    hipDeviceProp_t prop;
    int cus = 256;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        cus = prop.multiProcessorCount;
    return cus;      // one 8-wave workgroup per CU: its LDS holds the slice ring
}

template <int NCH, int NB, int WAVES = 8, int SPT = 2, int BLK = 1, int HO = 1, int KS = 1, bool SPLIT = false>
static hipError_t launch_wide_n(const ScanArgs &a, int grid, hipStream_t s) {
    const size_t lds = wide_lds_bytes(wide_ring(HO), KS * 2 * (NCH / SPT) * 1024, a.nq_tile, BLK, KS, SPLIT);
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_scan_p4_wide<NCH, NB, WAVES, SPT, BLK, HO, KS, SPLIT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((k_scan_p4_wide<NCH, NB, WAVES, SPT, BLK, HO, KS, SPLIT>), dim3(grid), dim3(WAVES * 64), lds, s, a);
    return hipGetLastError();
}

// Row lengths whose instance decodes half of a chunk through the LDS byte table: their weights
// come in the split order of k_scan_p4 (launch_build_p / launch_prep_p, `split`).
bool wide_weights_split(int nch) { return nch >= 12 && nch <= 24; }

// a.nq_tile = all queries of the launch (any number up to the chunk size), a.tables = their
// ceil(nq/32) weight tiles back to back, a.qscale / a.qbias / a.gtau indexed by query.
hipError_t launch_scan_p4_wide(const ScanArgs &a, int grid, hipStream_t s) {
    switch (a.nch) {
        // <chunks, B-operand registers, waves, slices per tile, blocks per wave, slices per hand-over>
        // One hand-over per tile (two slices) measured 2.5 to 5 % faster than one per slice in the
        // eight-wave forms with two slices per tile, and 2 % slower in the four-wave forms.
        case 2: return launch_wide_n<2, 2, 8, 1, 6>(a, grid, s);
        case 4: return launch_wide_n<4, 2, 8, 1, 4>(a, grid, s);
        case 6: return launch_wide_n<6, 2, 8, 1, 3>(a, grid, s);
        case 8: return launch_wide_n<8, 4, 8, 1, 2>(a, grid, s);
        case 10: return launch_wide_n<10, 2, 8, 2, 2, 2>(a, grid, s);
        case 12: return launch_wide_n<12, 2, 8, 2, 1, 2, 1, true>(a, grid, s);   // two blocks per wave would spill 21 registers
        case 14: return launch_wide_n<14, 2, 8, 2, 1, 2, 1, true>(a, grid, s);
        case 16: return launch_wide_n<16, 4, 8, 2, 1, 2, 1, true>(a, grid, s);
        case 18: return launch_wide_n<18, 2, 8, 2, 1, 2, 1, true>(a, grid, s);
        case 20: return launch_wide_n<20, 2, 8, 2, 1, 2, 1, true>(a, grid, s);   // (four operand registers in flight would spill one)
        case 22: return launch_wide_n<22, 2, 8, 2, 1, 2, 1, true>(a, grid, s);
        // 24 chunks (1536 dimensions): up to 1632 queries with the ring of five 24 KiB slices; longer
        // chunks (to 2048 queries: a block is then decoded once per 64 tiles instead of 32) with a
        // ring of nine 12 KiB slices handed over four at a time, which leaves the LDS for them
        case 24:
            if (a.nq_tile <= wide_max_queries_of(wide_ring(2), 24 * 1024, 1, 1, true)) return launch_wide_n<24, 2, 8, 2, 1, 2, 1, true>(a, grid, s);
            return launch_wide_n<24, 2, 8, 4, 1, 4, 1, true>(a, grid, s);
        case 28: return launch_wide_n<28, 2, 4, 4, 1>(a, grid, s);
        case 32: return launch_wide_n<32, 4, 4, 4, 1>(a, grid, s);
        case 36: return launch_wide_n<36, 2, 4, 4, 1>(a, grid, s);
        case 40: return launch_wide_n<40, 4, 4, 4, 1>(a, grid, s);
        case 44: return launch_wide_n<44, 2, 4, 4, 1>(a, grid, s);
        case 48: return launch_wide_n<48, 4, 4, 4, 1>(a, grid, s);
        // rows beyond one wave's registers, split over wave pairs: <chunks per wave, ..., slices of 4 chunks>
        case 56: return launch_wide_n<28, 2, 4, 7, 1, 1, 2>(a, grid, s);
        case 64: return launch_wide_n<32, 2, 4, 8, 1, 1, 2>(a, grid, s);
        case 72: return launch_wide_n<36, 2, 4, 9, 1, 1, 2>(a, grid, s);
        case 80: return launch_wide_n<40, 2, 4, 10, 1, 1, 2>(a, grid, s);
        case 88: return launch_wide_n<44, 2, 4, 11, 1, 1, 2>(a, grid, s);
        case 96: return launch_wide_n<48, 2, 4, 12, 1, 1, 2>(a, grid, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace tv
