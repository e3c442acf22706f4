// Device-side helpers shared by the scan, merge and select kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace tv {

// ===========================================================================
// Top-k bookkeeping shared by the scan kernels and the merge kernel.
// Total order: higher score first, ties to the lower slot
// (turbovec/src/search.rs:244-252 and :4285-4289).  Float compares make
// -0.0 and +0.0 tie, as partial_cmp does.
// ===========================================================================

__device__ __forceinline__ bool ranks_before(float s, uint32_t i, float s2, uint32_t i2) {
    return s > s2 || (s == s2 && i < i2);
}

// Monotone float -> signed int key (for atomicMax on thresholds).
__device__ __forceinline__ int order_key(float f) {
    const int b = __float_as_int(f);
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float order_unkey(int k) { return __int_as_float(k ^ ((k >> 31) & 0x7fffffff)); }
// order_key(-infinity): the threshold every real score passes.
constexpr int kTauInit = int(0x807fffffu);

// A lane-private unsorted list of up to k entries living in LDS at
// ls/li[entry * stride + slot_of_lane]; the lane keeps its size, and its worst
// entry (score, index, position) in registers.
struct LaneList {
    int cnt;
    float worst_s;
    uint32_t worst_i;
    int worst_pos;
};

__device__ __forceinline__ void list_rescan(LaneList &L, const float *ls, const uint32_t *li, int stride, int me,
                                            int k) {
    float ws = ls[me];
    uint32_t wi = li[me];
    int wp = 0;
    for (int e = 1; e < k; ++e) {
        const float s = ls[e * stride + me];
        const uint32_t i = li[e * stride + me];
        if (ranks_before(ws, wi, s, i)) { ws = s; wi = i; wp = e; }
    }
    L.worst_s = ws; L.worst_i = wi; L.worst_pos = wp;
}

// Returns true when the list is full after the call and its worst entry changed.
__device__ __forceinline__ bool list_offer(LaneList &L, float *ls, uint32_t *li, int stride, int me, int k, float s,
                                           uint32_t idx) {
    if (L.cnt < k) {
        ls[L.cnt * stride + me] = s;
        li[L.cnt * stride + me] = idx;
        ++L.cnt;
        if (L.cnt == k) { list_rescan(L, ls, li, stride, me, k); return true; }
        return false;
    }
    if (!ranks_before(s, idx, L.worst_s, L.worst_i)) return false;
    ls[L.worst_pos * stride + me] = s;
    li[L.worst_pos * stride + me] = idx;
    list_rescan(L, ls, li, stride, me, k);
    return true;
}

__device__ __forceinline__ uint64_t sort_key(float s, uint32_t idx) {
    // high word: order key of the score with -0.0 folded onto +0.0 (they tie);
    // low word: inverted slot so that the lower slot sorts first, plus one bit
    // remembering a negative zero so the emitted score keeps its sign bit.
    const bool negzero = __float_as_uint(s) == 0x80000000u;
    const float canon = negzero ? 0.0f : s;
    const uint32_t hi = uint32_t(order_key(canon)) ^ 0x80000000u;
    const uint32_t lo = ((0x7fffffffu - idx) << 1) | (negzero ? 1u : 0u);
    return (uint64_t(hi) << 32) | lo;
}
__device__ __forceinline__ void sort_unkey(uint64_t key, float &s, uint32_t &idx) {
    const uint32_t hi = uint32_t(key >> 32), lo = uint32_t(key);
    s = order_unkey(int(hi ^ 0x80000000u));
    if (lo & 1u) s = -0.0f;
    idx = 0x7fffffffu - (lo >> 1);
}


typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------------------
// Hand-placed code loads.  The vector-memory counter retires in order, and the
// compiler's own wait placement is decided per merge point of the control flow,
// which for a software-pipelined stream ends up waiting on the burst it has
// just issued.  These loads are invisible to that pass: the kernel states how
// many younger loads may stay in flight where it consumes a register
// (wait_vm<N>).  Loads the compiler issues itself only make its own waits
// stricter, never looser, because a count is an upper bound on what may remain.
// ---------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16 bytes of the code stream: read once per pass, so loaded with the non-temporal hint -- the
// stream then does not turn the caches over, and the read rate rises by about a tenth.
__device__ __forceinline__ uint4 load_stream16(const uint4 *p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

template <int OFF>
__device__ __forceinline__ void load16_async(u32x4 &dst, const void *p) {
    asm volatile("global_load_dwordx4 %0, %1, off offset:%2 nt" : "=v"(dst) : "v"(p), "n"(OFF));
}
__device__ __forceinline__ void load4_async(float &dst, const void *p) {
    asm volatile("global_load_dword %0, %1, off" : "=v"(dst) : "v"(p));
}
template <int N>
__device__ __forceinline__ void wait_vm(u32x4 &r) {
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_vm(float &r) {
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r) : "n"(N));
}

// Four packed nibbles (one per byte, values 0..15) -> four int8 levels.
// v_perm_b32 looks up 8 table bytes; selectors >= 13 give 0xff, so each half
// of the 16-entry table is looked up with the other half's nibbles pushed out
// of range, and the two results are ANDed.
__device__ __forceinline__ uint32_t levels_of(uint32_t nib, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
    const uint32_t selA = nib + (nib & 0x08080808u);  // 0..7 stay, 8..15 -> 16..23
    const uint32_t selB = selA ^ 0x10101010u;         // 0..7 -> 16..23, 16..23 -> 0..7
    return __builtin_amdgcn_perm(t1, t0, selA) & __builtin_amdgcn_perm(t3, t2, selB);
}

// Largest value of v over the wave (all 64 lanes active), in every lane: four butterfly steps inside
// each row of 16 lanes on the data-parallel path (no LDS), then the four row results through lane
// reads.
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
    v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0xB1, 0xf, 0xf, false)));    // quad_perm [1,0,3,2]
    v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x4E, 0xf, 0xf, false)));    // quad_perm [2,3,0,1]
    v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x141, 0xf, 0xf, false)));   // row_half_mirror
    v = max(v, uint32_t(__builtin_amdgcn_update_dpp(0, int(v), 0x140, 0xf, 0xf, false)));   // row_mirror
    const uint32_t a = uint32_t(__builtin_amdgcn_readlane(int(v), 0)), b = uint32_t(__builtin_amdgcn_readlane(int(v), 16));
    const uint32_t c = uint32_t(__builtin_amdgcn_readlane(int(v), 32)), d = uint32_t(__builtin_amdgcn_readlane(int(v), 48));
    return max(max(a, b), max(c, d));
}

// The code byte -> (level of its low nibble, level of its high nibble) table the permute-dot scans
// keep at the start of their LDS: 256 entries of two int8 levels.
constexpr int kDecodeBytes = 512;

// A 16-bit LDS load, zero-extended, requested without telling the compiler's wait-count
// bookkeeping (the caller's `s_waitcnt lgkmcnt(N)`, tied to the destinations, is the matching
// wait).  The loads that fill one half of a register and keep the other are no use here: with
// ECC-protected register files they clear it.
__device__ __forceinline__ void lds_u16(uint32_t &dst, uint32_t addr) {
    asm volatile("ds_read_u16 %0, %1" : "=v"(dst) : "v"(addr));
}
// 2 * byte E of x: the offset of that code byte's table entry.
template <int E>
__device__ __forceinline__ uint32_t byte_x2(uint32_t x) {
    uint32_t r;
    if (E == 0) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(1u), "v"(x));
    if (E == 1) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(1u), "v"(x));
    if (E == 2) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(1u), "v"(x));
    if (E == 3) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(1u), "v"(x));
    return r;
}

// A conditional launch: true when the flag it depends on says there is nothing to do.  The flag is
// uniform over the grid and written by an earlier launch of the same stream.
__device__ __forceinline__ bool launch_switched_off(const uint32_t *run_if) {
    return run_if != nullptr && *reinterpret_cast<const volatile uint32_t *>(run_if) == 0u;
}

// Compile-time loop: f(IntC<0>{}), ..., f(IntC<N-1>{}), for bodies that index register arrays.
template <int V> struct IntC { static constexpr int value = V; };
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(IntC<I>{});
        static_for<N, I + 1>(f);
    }
}

}  // namespace tv
