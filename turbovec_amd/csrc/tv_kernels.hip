// HIP kernels of the turbovec search path for gfx950 (MI355X).
//
// Compiled with -ffp-contract=off: every float expression keeps the separate
// multiplies and adds the reference performs, and fmaf appears only where the
// reference fuses.
#include "tv_internal.h"
#include "tv_device.h"

#include <cfloat>
#include <climits>
#include <cstdlib>

namespace tv {



// ===========================================================================
// Layout transforms between the persisted sequential-blocked layout
// (turbovec/src/pack.rs:336-361) and the native chunked layout.
// ===========================================================================

// One workgroup per (block, chunk): a 1 KiB tile of 32 groups x 32 lanes is
// transposed through LDS so both sides move as dwords.
__global__ __launch_bounds__(256) void k_seq_to_native(const uint8_t *__restrict__ seq, uint8_t *__restrict__ nat,
                                                       int G, int nch, size_t first_block) {
    __shared__ uint8_t tile[32 * 36];  // [group][lane], rows padded to 36 bytes
    const size_t b = first_block + blockIdx.x / nch;
    const int c = blockIdx.x % nch;
    const int t = threadIdx.x;
    {   // read: dword t covers group gl = t/8, lanes 4*(t%8)..+3
        const int gl = t >> 3, l4 = (t & 7) * 4;
        const int g = c * 32 + gl;
        uint32_t v = 0;
        if (g < G) v = *reinterpret_cast<const uint32_t *>(seq + ((b - first_block) * size_t(G) + g) * 32 + l4);
        *reinterpret_cast<uint32_t *>(tile + gl * 36 + l4) = v;
    }
    __syncthreads();
    {   // write: dword t of the chunk = lane l = t/4 (h = l/32, i = l%32), bytes j0..j0+3
        const int l = t >> 2, j0 = (t & 3) * 4;
        const int h = l >> 5, i = l & 31;
        uint32_t v = 0;
        for (int j = 0; j < 4; ++j) v |= uint32_t(tile[(16 * h + j0 + j) * 36 + i]) << (8 * j);
        *reinterpret_cast<uint32_t *>(nat + (b * size_t(nch) + c) * 1024 + size_t(t) * 4) = v;
    }
}

__global__ __launch_bounds__(256) void k_native_to_seq(const uint8_t *__restrict__ nat, uint8_t *__restrict__ seq,
                                                       int G, int nch, size_t first_block) {
    __shared__ uint8_t tile[32 * 36];
    const size_t b = first_block + blockIdx.x / nch;
    const int c = blockIdx.x % nch;
    const int t = threadIdx.x;
    {
        const int l = t >> 2, j0 = (t & 3) * 4;
        const int h = l >> 5, i = l & 31;
        const uint32_t v = *reinterpret_cast<const uint32_t *>(nat + (b * size_t(nch) + c) * 1024 + size_t(t) * 4);
        for (int j = 0; j < 4; ++j) tile[(16 * h + j0 + j) * 36 + i] = uint8_t(v >> (8 * j));
    }
    __syncthreads();
    {
        const int gl = t >> 3, l4 = (t & 7) * 4;
        const int g = c * 32 + gl;
        if (g < G)
            *reinterpret_cast<uint32_t *>(seq + ((b - first_block) * size_t(G) + g) * 32 + l4) =
                *reinterpret_cast<const uint32_t *>(tile + gl * 36 + l4);
    }
}

__device__ __forceinline__ size_t native_byte_index(size_t v, int g, int nch) {
    const size_t b = v >> 5;
    const int i = int(v & 31);
    return ((b * size_t(nch) + size_t(g >> 5)) * 64 + size_t(((g & 31) >> 4) * 32 + i)) * 16 + size_t(g & 15);
}

// rows[r*G + g] -> lane of vector old_n + r (turbovec/src/pack.rs:211-233 append_lanes).
__global__ void k_append_rows(const uint8_t *__restrict__ rows, uint8_t *__restrict__ nat, int G, int nch,
                              size_t old_n, size_t n_new) {
    const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= n_new * size_t(G)) return;
    const size_t r = idx / G;
    const int g = int(idx % G);
    nat[native_byte_index(old_n + r, g, nch)] = rows[idx];
}

// turbovec/src/lib.rs:2964-3003: move_lane(last -> idx), zero_lane(last), scale move.
__global__ void k_move_lane(uint8_t *__restrict__ nat, float *__restrict__ scales, int G, int nch, size_t src,
                            size_t dst) {
    const int g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g < G) {
        const size_t s = native_byte_index(src, g, nch);
        if (src != dst) nat[native_byte_index(dst, g, nch)] = nat[s];
        nat[s] = 0;
    }
    if (g == 0) {
        if (src != dst) scales[dst] = scales[src];
        scales[src] = 0.0f;
    }
}

// Queries whose candidates overflowed, packed for one more full scan: row r of the packed batch
// is query rows[r] of the chunk, its floor the raised one k_final left for it, placed where the
// scan kernels read the floors of tile r / tile_q.
__global__ __launch_bounds__(256) void k_gather_redo(const float *__restrict__ q, const uint32_t *__restrict__ rows,
                                                     const int *__restrict__ raised, int dim, int tile_q,
                                                     float *__restrict__ q_out, int *__restrict__ tau_out) {
    const uint32_t r = blockIdx.x, o = rows[r];
    for (int i = threadIdx.x; i < dim; i += 256) q_out[size_t(r) * dim + i] = q[size_t(o) * dim + i];
    if (threadIdx.x == 0) tau_out[(r / tile_q) * kQTile + r % tile_q] = raised[o];
}

__global__ void k_fill_i32(int *p, int v, size_t n) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ===========================================================================
// Query preparation
// ===========================================================================

// turbovec/src/rotation.rs:265-320 (apply_with_scratch) + :964-982 (wht_block_scalar).
// One workgroup per query row; both rounds run in LDS.  Every output element is
// produced by the same IEEE adds, subtracts and multiplies, in the same
// operand pairing, as the scalar butterfly, so the result is bit-identical.
__global__ __launch_bounds__(256) void k_rotate(const float *__restrict__ q, float *__restrict__ out,
                                                const float *__restrict__ signs,
                                                const uint32_t *__restrict__ perms, int dim, int block,
                                                float inv_sqrt_block) {
    extern __shared__ float rot_lds[];
    float *A = rot_lds;
    float *B = rot_lds + dim;
    const float *src = q + size_t(blockIdx.x) * dim;
    const int t = threadIdx.x;
    for (int i = t; i < dim; i += 256) A[i] = src[perms[i]] * signs[i];
    __syncthreads();
    for (int len = 1; len < block; len <<= 1) {
        for (int p = t; p < dim / 2; p += 256) {
            const int j = 2 * p - (p & (len - 1));
            const float a = A[j], b = A[j + len];
            A[j] = a + b;
            A[j + len] = a - b;
        }
        __syncthreads();
    }
    // the 1/sqrt(B) scale of round 0 rides the round-1 gather: (x * inv) * sign
    for (int i = t; i < dim; i += 256) B[i] = (A[perms[dim + i]] * inv_sqrt_block) * signs[dim + i];
    __syncthreads();
    for (int len = 1; len < block; len <<= 1) {
        for (int p = t; p < dim / 2; p += 256) {
            const int j = 2 * p - (p & (len - 1));
            const float a = B[j], b = B[j + len];
            B[j] = a + b;
            B[j + len] = a - b;
        }
        __syncthreads();
    }
    float *dst = out + size_t(blockIdx.x) * dim;
    for (int i = t; i < dim; i += 256) dst[i] = B[i] * inv_sqrt_block;
}

// turbovec/src/search.rs:3154-3186 calibrate_queries.  The f64 bias sum is
// sequential over d, so one thread carries it.
__global__ __launch_bounds__(256) void k_calibrate(const float *__restrict__ qrot, float *__restrict__ qcal,
                                                   float *__restrict__ bias_corr,
                                                   const float *__restrict__ shift,
                                                   const float *__restrict__ scale, int dim) {
    const float *src = qrot + size_t(blockIdx.x) * dim;
    float *dst = qcal + size_t(blockIdx.x) * dim;
    for (int i = threadIdx.x; i < dim; i += 256) dst[i] = src[i] / scale[i];
    if (threadIdx.x == 0) {
        double bc = 0.0;
        for (int d = 0; d < dim; ++d) bc -= double(src[d]) * double(shift[d]);
        bias_corr[blockIdx.x] = float(bc);
    }
}

__device__ __forceinline__ float block_max_256(float v, float *red) {
    // exact: max is order-free
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    return v;
}

__device__ __forceinline__ float clamp_round_i8(float v) {
    // Rust f32::round is half-away-from-zero, like roundf; then clamp(-127, 127)
    v = roundf(v);
    return v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
}

// turbovec/src/search.rs:2806-2846 build_permute_dot, emitting the weights in
// the MFMA B-fragment order of the scan.  Plane order (the batched scans, whose
// decode yields one A operand of low nibbles and one of high nibbles per chunk):
// for query tile t, chunk c and nibble plane p (0 = low nibble = odd dimension,
// 1 = high nibble = even dimension) a 1 KiB fragment whose lane (h*32 + n) holds
// the 16 weights of query n for groups 32c + 16h .. +15.  Split order (k_scan_p4,
// which decodes the first 8 code bytes of a lane on the vector ALU, four at a
// time, and looks the other 8 up whole, both levels of a byte side by side):
// fragment 0 of chunk c holds, in lane (h*32 + n), for e = 0..7, the plane-p
// weight of group 32c + 16h + e at byte 8*(e/4) + 4p + e%4; fragment 1 the
// plane-p weight of group 32c + 16h + 8 + e at byte 2e + p.
__device__ __forceinline__ size_t wfrag_offset(int g, int n, int plane, bool split) {
    const size_t lane16 = size_t(((g & 31) >> 4) * 32 + n) * 16;
    if (split) {
        const int e = g & 7;
        const int at = (g & 8) ? 2 * e + plane : 8 * (e >> 2) + 4 * plane + (e & 3);
        return size_t(g >> 5) * 2048 + size_t((g & 15) >> 3) * 1024 + lane16 + size_t(at);
    }
    return size_t(g >> 5) * 2048 + size_t(plane) * 1024 + lane16 + size_t(g & 15);
}

__global__ __launch_bounds__(256) void k_build_p(const float *__restrict__ qcal,
                                                 const float *__restrict__ bias_corr,
                                                 uint8_t *__restrict__ wfrag, float *__restrict__ qscale,
                                                 float *__restrict__ qbias, int dim, int G, int nch, float cs,
                                                 size_t nq, bool split) {
    __shared__ float red[4];
    const size_t qi = blockIdx.x;
    const size_t tile = qi / kQTile;
    const int n = int(qi % kQTile);
    uint8_t *base = wfrag + tile * size_t(nch) * 2048;
    const int t = threadIdx.x;
    if (qi >= nq) {  // padding query of the last tile: zero weights
        for (int g = t; g < nch * 32; g += 256) {
            base[wfrag_offset(g, n, 0, split)] = 0;
            base[wfrag_offset(g, n, 1, split)] = 0;
        }
        if (t == 0) { qscale[qi] = 0.0f; qbias[qi] = 0.0f; }
        return;
    }
    const float *q = qcal + qi * size_t(dim);
    float m = 0.0f;
    for (int d = t; d < dim; d += 256) m = fmaxf(m, fabsf(q[d]));
    const float qmax = block_max_256(m, red);
    float qs = qmax / 127.0f, inv_qs;
    if (qs >= FLT_MIN) inv_qs = 1.0f / qs; else { qs = 1.0f; inv_qs = 1.0f; }
    for (int g = t; g < nch * 32; g += 256) {
        int8_t lo = 0, hi = 0;
        if (g < G) {
            lo = int8_t(clamp_round_i8(q[2 * g + 1] * inv_qs));
            hi = int8_t(clamp_round_i8(q[2 * g] * inv_qs));
        }
        base[wfrag_offset(g, n, 0, split)] = uint8_t(lo);
        base[wfrag_offset(g, n, 1, split)] = uint8_t(hi);
    }
    if (t == 0) {
        qscale[qi] = cs * qs;
        qbias[qi] = 0.0f + (bias_corr ? bias_corr[qi] : 0.0f);
    }
}

// Query preparation of the permute-dot mode in one launch, one workgroup per query: k_rotate,
// k_calibrate and k_build_p back to back with the row kept in LDS between them -- the same
// operations on the same values in the same order, so the same bits (search.rs:3237-3269).  A
// single query's preparation is three dependent launches' worth of latency otherwise.
__global__ __launch_bounds__(256) void k_prep_p(const float *__restrict__ q, const float *__restrict__ signs,
                                                const uint32_t *__restrict__ perms, int dim, int block,
                                                float inv_sqrt_block, const float *__restrict__ shift,
                                                const float *__restrict__ scale, uint8_t *__restrict__ wfrag,
                                                float *__restrict__ qscale, float *__restrict__ qbias, int G, int nch,
                                                float cs, size_t nq, bool split) {
    extern __shared__ float rot_lds[];
    __shared__ float red[4];
    __shared__ float s_bias;
    float *A = rot_lds;
    float *B = rot_lds + dim;
    const size_t qi = blockIdx.x;
    const size_t tile = qi / kQTile;
    const int n = int(qi % kQTile);
    uint8_t *base = wfrag + tile * size_t(nch) * 2048;
    const int t = threadIdx.x;
    if (qi >= nq) {  // padding query of the last tile: zero weights
        for (int g = t; g < nch * 32; g += 256) {
            base[wfrag_offset(g, n, 0, split)] = 0;
            base[wfrag_offset(g, n, 1, split)] = 0;
        }
        if (t == 0) { qscale[qi] = 0.0f; qbias[qi] = 0.0f; }
        return;
    }
    const float *src = q + qi * size_t(dim);
    for (int i = t; i < dim; i += 256) A[i] = src[perms[i]] * signs[i];
    __syncthreads();
    for (int len = 1; len < block; len <<= 1) {
        for (int p = t; p < dim / 2; p += 256) {
            const int j = 2 * p - (p & (len - 1));
            const float a = A[j], b = A[j + len];
            A[j] = a + b;
            A[j + len] = a - b;
        }
        __syncthreads();
    }
    for (int i = t; i < dim; i += 256) B[i] = (A[perms[dim + i]] * inv_sqrt_block) * signs[dim + i];
    __syncthreads();
    for (int len = 1; len < block; len <<= 1) {
        for (int p = t; p < dim / 2; p += 256) {
            const int j = 2 * p - (p & (len - 1));
            const float a = B[j], b = B[j + len];
            B[j] = a + b;
            B[j + len] = a - b;
        }
        __syncthreads();
    }
    // the rotated row (k_rotate's output) into A; with a TQ+ pair, k_calibrate's output over it
    for (int i = t; i < dim; i += 256) A[i] = B[i] * inv_sqrt_block;
    __syncthreads();
    if (scale != nullptr) {
        if (t == 0) {
            double bc = 0.0;
            for (int d = 0; d < dim; ++d) bc -= double(A[d]) * double(shift[d]);
            s_bias = float(bc);
        }
        __syncthreads();
        for (int i = t; i < dim; i += 256) A[i] = A[i] / scale[i];
        __syncthreads();
    }
    const float *qc = A;
    float m = 0.0f;
    for (int d = t; d < dim; d += 256) m = fmaxf(m, fabsf(qc[d]));
    const float qmax = block_max_256(m, red);
    float qs = qmax / 127.0f, inv_qs;
    if (qs >= FLT_MIN) inv_qs = 1.0f / qs; else { qs = 1.0f; inv_qs = 1.0f; }
    for (int g = t; g < nch * 32; g += 256) {
        int8_t lo = 0, hi = 0;
        if (g < G) {
            lo = int8_t(clamp_round_i8(qc[2 * g + 1] * inv_qs));
            hi = int8_t(clamp_round_i8(qc[2 * g] * inv_qs));
        }
        base[wfrag_offset(g, n, 0, split)] = uint8_t(lo);
        base[wfrag_offset(g, n, 1, split)] = uint8_t(hi);
    }
    if (t == 0) {
        qscale[qi] = cs * qs;
        qbias[qi] = 0.0f + (scale != nullptr ? s_bias : 0.0f);
    }
}

// turbovec/src/search.rs:2856-2994 build_query_neon_lut_from_slice.  Output per
// query: nch*32 rows of 32 bytes, row g = [16 entries indexed by the byte's HIGH
// nibble (the group's first dimensions) | 16 entries indexed by the LOW nibble];
// rows of padding groups are zero.
template <int BITS>
__device__ __forceinline__ float lut_entry(const float *q, const float *cen, int dim_start, int sub, int nv) {
    constexpr int cpb = 8 / BITS, cpn = cpb / 2;
    constexpr unsigned code_mask = (1u << BITS) - 1;
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < cpn; ++c) {
        const int sh = (cpn - 1 - c) * BITS;
        const unsigned code = (unsigned(nv) >> sh) & code_mask;
        s += q[dim_start + sub * cpn + c] * cen[code];
    }
    return s;
}

template <int BITS>
__global__ __launch_bounds__(256) void k_build_lut(const float *__restrict__ qcal,
                                                   const float *__restrict__ bias_corr,
                                                   const float *__restrict__ centroids,
                                                   uint8_t *__restrict__ lut, float *__restrict__ qscale,
                                                   float *__restrict__ qbias, int dim, int G, int nch, size_t nq) {
    extern __shared__ float lut_lds[];  // mins: 2*G floats
    __shared__ float red[4];
    __shared__ float cen[16];
    constexpr int cpb = 8 / BITS;
    const size_t qi = blockIdx.x;
    uint8_t *dst = lut + qi * size_t(nch) * 1024;
    const int t = threadIdx.x;
    if (qi >= nq) {
        for (int i = t; i < nch * 256; i += 256) reinterpret_cast<uint32_t *>(dst)[i] = 0;
        if (t == 0) { qscale[qi] = 0.0f; qbias[qi] = 0.0f; }
        return;
    }
    if (t < (1 << BITS)) cen[t] = centroids[t];
    __syncthreads();
    const float *q = qcal + qi * size_t(dim);
    float span = 0.0f;
    for (int g = t; g < G; g += 256) {
        for (int sub = 0; sub < 2; ++sub) {
            float mn = FLT_MAX, mx = -FLT_MAX;
            for (int nv = 0; nv < 16; ++nv) {
                const float s = lut_entry<BITS>(q, cen, g * cpb, sub, nv);
                if (s < mn) mn = s;
                if (s > mx) mx = s;
            }
            lut_lds[2 * g + sub] = mn;
            span = fmaxf(span, mx - mn);
        }
    }
    const float max_span = block_max_256(span, red);  // also orders the lut_lds writes
    float scale = max_span > 0.0f ? max_span / 127.0f : 1.0f, inv_scale;
    if (scale >= FLT_MIN) inv_scale = 1.0f / scale; else { scale = 1.0f; inv_scale = 1.0f; }
    if (t == 0) {
        float bias = 0.0f;  // sequential f32 sum over groups, inner add first (search.rs:2910)
        for (int g = 0; g < G; ++g) bias += lut_lds[2 * g] + lut_lds[2 * g + 1];
        qscale[qi] = scale;
        qbias[qi] = bias + (bias_corr ? bias_corr[qi] : 0.0f);
    }
    for (int g = t; g < nch * 32; g += 256) {
        uint32_t w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (g < G) {
            for (int sub = 0; sub < 2; ++sub) {
                const float mn = lut_lds[2 * g + sub];
                for (int nv = 0; nv < 16; ++nv) {
                    float v = roundf((lut_entry<BITS>(q, cen, g * cpb, sub, nv) - mn) * inv_scale);
                    v = v < 0.0f ? 0.0f : (v > 127.0f ? 127.0f : v);
                    w[sub * 4 + nv / 4] |= uint32_t(uint8_t(v)) << (8 * (nv & 3));
                }
            }
        }
        uint4 *o = reinterpret_cast<uint4 *>(dst + size_t(g) * 32);
        o[0] = make_uint4(w[0], w[1], w[2], w[3]);
        o[1] = make_uint4(w[4], w[5], w[6], w[7]);
    }
}

// ===========================================================================
// Scan, score mode P: 4-bit codes -> int8 codebook levels -> i8 MFMA against
// int8 query weights (turbovec/src/search.rs:1392-1567 computes the same
// integers with vpdpbusd).  acc = sum_d w[d] * level[code[d]], exact in i32;
// score = fma(f32(acc), scale, bias) * vec_scale (search.rs:1519-1524).
//
// k_scan_p4 decodes half of a chunk through LDS: a 256-entry table maps a code
// byte to the two levels of its nibbles (low nibble's in the low byte); two
// entries make one dword of an A operand -- one shift (the byte's table
// offset), one LDS read and half a merge per code byte, against 3.75
// vector-ALU instructions per byte for the in-register lookup, which alone held
// this kernel below the HBM stream (as does one LDS instruction per byte alone).
// The table sits at the start of the kernel's LDS (there is no static
// allocation before it), so a byte's offset is its address.
// ===========================================================================
// 16 bytes of LDS per lane, requested like the table entries (lds_u16): behind the compiler's
// wait-count bookkeeping, lds_settle being the matching wait.
template <int OFF>
__device__ __forceinline__ void lds_b128(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst) : "v"(addr), "n"(OFF));
}
// Hold until at most N LDS requests younger than those feeding e, o, w0 and w1 are outstanding.
template <int N>
__device__ __forceinline__ void lds_settle(uint32_t (&e)[4], uint32_t (&o)[4], v4i &w0, v4i &w1) {
    asm volatile("s_waitcnt lgkmcnt(%10)" : "+v"(e[0]), "+v"(e[1]), "+v"(e[2]), "+v"(e[3]), "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(w0), "+v"(w1) : "n"(N));
}

// The same with a run-time address, and a full wait tied to the registers a step is about to use.
__device__ __forceinline__ void lds_b128_at(v4i &dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1" : "=&v"(dst) : "v"(addr));
}
// (the same for two table dwords)
template <int NT>
__device__ __forceinline__ void lds_settle_all(uint32_t (&e)[2], uint32_t (&o)[2], v4i (&w)[NT]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e[0]), "+v"(e[1]), "+v"(o[0]), "+v"(o[1]));
#pragma unroll
    for (int t = 0; t < NT; ++t) asm volatile("" : "+v"(w[t]));
}
template <int NT>
__device__ __forceinline__ void lds_settle_all(uint32_t (&e)[4], uint32_t (&o)[4], v4i (&w)[NT]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e[0]), "+v"(e[1]), "+v"(e[2]), "+v"(e[3]), "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]));
#pragma unroll
    for (int t = 0; t < NT; ++t) asm volatile("" : "+v"(w[t]));
}

// n16 16-byte words from global memory into LDS by a workgroup of THREADS, twelve loads per thread
// in flight at a time: a scan launch that reads a block or two per wave (a sampling level, a
// small index) is as long as its set-up, and word after word the copy is a chain of trips to L2.
template <int THREADS>
__device__ __forceinline__ void stage_to_lds(uint4 *dst, const uint4 *src, int n16, int tid) {
    constexpr int kBatch = 12;
    for (int i0 = tid; i0 < n16; i0 += THREADS * kBatch) {
        uint4 tmp[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int i = i0 + u * THREADS;
            tmp[u] = i < n16 ? src[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const int i = i0 + u * THREADS;
            if (i < n16) dst[i] = tmp[u];
        }
    }
}

template <int U, int MODE, bool W_LDS, int THREADS = kScanThreads>
__global__ __launch_bounds__(THREADS) void k_scan_p4(ScanArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr bool LISTS = MODE == kModeLists, DUMP = MODE == kModeDump, BEST = MODE == kModeBest;
    constexpr bool APPEND = MODE == kModeAppend || BEST;     // both fill the candidate segments
    if (APPEND && launch_switched_off(a.run_if)) return;
    const int nch = a.nch, k = a.k;
    uint8_t *sW = smem + kDecodeBytes;
    const size_t w_bytes = kDecodeBytes + (W_LDS ? size_t(nch) * 2048 : 0);
    float *ls = reinterpret_cast<float *>(smem + w_bytes);
    uint32_t *li = reinterpret_cast<uint32_t *>(ls + (LISTS ? k * THREADS : 0));
    int *stau = reinterpret_cast<int *>(li + (LISTS ? k * THREADS : 0));
    uint32_t *scnt = reinterpret_cast<uint32_t *>(stau);  // append mode: candidates per query of this workgroup

    // A workgroup of more than four waves is GROUPS four-wave groups that share the weights in LDS
    // and are, in every other respect, workgroups vb of a launch of a.vgrid four-wave workgroups:
    // the same blocks per wave, a candidate segment per group.
    constexpr int GROUPS = THREADS / kScanThreads;
    static_assert(THREADS % kScanThreads == 0 && (GROUPS == 1 || APPEND), "wave groups are an append-mode form");
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = (tid >> 6) % (kScanThreads / 64);
    const int qn = lane & 31, h = lane >> 5;
    const uint32_t vgrid = GROUPS > 1 ? a.vgrid : gridDim.x;
    const uint32_t vb = GROUPS > 1 ? blockIdx.x * GROUPS + uint32_t(tid) / kScanThreads : blockIdx.x;
    if (GROUPS > 1) scnt += (tid / kScanThreads) * kQTile;

    // Logical blocks j = 0..nj-1 stand for physical blocks j*step (step > 1 samples the index).
    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;
    const uint32_t total_waves = vgrid * (kScanThreads / 64);
    const uint32_t gw = wave * vgrid + vb;  // consecutive blocks go to different workgroups
    // Blocks are dealt round-robin to the waves of the grid: wave gw takes logical blocks gw,
    // gw + total_waves, ...  Neighbouring rows (clustered data, contiguous allowlists) then spread
    // over all workgroups instead of piling into one.
    const uint32_t j_begin = gw, j_end = (GROUPS > 1 && vb >= vgrid) ? 0u : nj;   // (a group beyond the launch's last has no blocks)
    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes) + lane;

    // first block with at least one allowed slot (search.rs:3015-3029)
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

    // the wave's first codes are on their way from HBM while the workgroup sets up its LDS
    uint32_t j = live_from(j_begin);
    uint4 buf[U];
    if (j < j_end) {
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_stream16(&codes[(size_t(j) * step * nch + u) * 64]);
    }

    if (W_LDS) stage_to_lds<THREADS>(reinterpret_cast<uint4 *>(sW), reinterpret_cast<const uint4 *>(a.tables), nch * 128, tid);
    for (int b = tid; b < 256; b += THREADS) {
        const uint32_t lo = (a.lv[(b & 15) >> 2] >> (8 * (b & 3))) & 0xffu;
        const uint32_t hi = (a.lv[b >> 6] >> (8 * ((b >> 4) & 3))) & 0xffu;
        reinterpret_cast<uint16_t *>(smem)[b] = uint16_t(lo | (hi << 8));
    }
    if (LISTS && tid < kQTile) stau[tid] = a.gtau[tid];
    if (APPEND && (tid % kScanThreads) < kQTile) scnt[tid % kScanThreads] = 0u;
    __syncthreads();

    const bool active = qn < a.nq_tile;
    const float qs = active ? a.qscale[qn] : 0.0f;
    const float qb = active ? a.qbias[qn] : 0.0f;
    const uint32_t t0 = a.lv[0], t1 = a.lv[1], t2 = a.lv[2], t3 = a.lv[3];
    // append mode: a fixed per-query floor; NaN for idle lanes so no compare passes
    const float tau_fixed = (APPEND && !BEST) ? (active ? order_unkey(a.gtau[qn]) : __int_as_float(0x7fc00000)) : 0.0f;

    LaneList L{0, 0.0f, 0u, 0};
    const uint4 *wglob = reinterpret_cast<const uint4 *>(a.tables) + lane;

    while (j < j_end) {
        const uint32_t nj_live = live_from(j + total_waves);
        const uint32_t b = j * step;
        v16i acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        for (int c0 = 0; c0 < nch; c0 += U) {
            // the next U chunks (of this block, or the head of the next one) are requested as one
            // contiguous burst before the current U are consumed
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
            // A chunk gives two A operands.  The first, from code bytes 0..7 of the lane, is decoded
            // on the vector ALU: dwords (low-nibble levels of bytes 0..3, high-nibble levels of bytes
            // 0..3, the same for bytes 4..7).  The second, from bytes 8..15, through the byte table:
            // dword r from bytes 8+2r (low half) and 9+2r (high half), each as its (low nibble, high
            // nibble) pair of levels.  Either unit alone is slower than the HBM stream (3.75 ALU
            // instructions per byte; one LDS instruction per byte); half each fits under it.  The
            // LDS requests of chunk u+1 are issued before chunk u is waited for.
            uint32_t e[2][4], o[2][4];
            v4i bw0[2], bw1[2];
            const uint32_t w_addr = uint32_t(kDecodeBytes + c0 * 2048 + lane * 16);
            auto request = [&](auto uc) {
                constexpr int u = decltype(uc)::value, p = u & 1;
                if (W_LDS) {
                    lds_b128<u * 2048>(bw0[p], w_addr);
                } else {
                    const uint4 w = wglob[(size_t(c0 + u) * 2) * 64];
                    bw0[p] = v4i{int(w.x), int(w.y), int(w.z), int(w.w)};
                }
                const uint32_t xa = cur[u].z, xb = cur[u].w;
                lds_u16(e[p][0], byte_x2<0>(xa)); lds_u16(o[p][0], byte_x2<1>(xa));
                lds_u16(e[p][1], byte_x2<2>(xa)); lds_u16(o[p][1], byte_x2<3>(xa));
                lds_u16(e[p][2], byte_x2<0>(xb)); lds_u16(o[p][2], byte_x2<1>(xb));
                lds_u16(e[p][3], byte_x2<2>(xb)); lds_u16(o[p][3], byte_x2<3>(xb));
                if (W_LDS) {
                    lds_b128<u * 2048 + 1024>(bw1[p], w_addr);
                } else {
                    const uint4 w = wglob[(size_t(c0 + u) * 2 + 1) * 64];
                    bw1[p] = v4i{int(w.x), int(w.y), int(w.z), int(w.w)};
                }
            };
            request(IntC<0>{});
            static_for<U>([&](auto uc) {
                constexpr int u = decltype(uc)::value, p = u & 1;
                if constexpr (u + 1 < U) request(IntC<u + 1>{});
                const v4i a0 = {int(levels_of(cur[u].x & 0x0f0f0f0fu, t0, t1, t2, t3)),
                                int(levels_of((cur[u].x >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3)),
                                int(levels_of(cur[u].y & 0x0f0f0f0fu, t0, t1, t2, t3)),
                                int(levels_of((cur[u].y >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3))};
                if constexpr (u + 1 < U) lds_settle<W_LDS ? 10 : 8>(e[p], o[p], bw0[p], bw1[p]);
                else lds_settle<0>(e[p], o[p], bw0[p], bw1[p]);
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, bw0[p], acc, 0, 0, 0);
                const v4i a1 = {int(e[p][0] | (o[p][0] << 16)), int(e[p][1] | (o[p][1] << 16)),
                                int(e[p][2] | (o[p][2] << 16)), int(e[p][3] | (o[p][3] << 16))};
                acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, bw1[p], acc, 0, 0, 0);
            });
        }

        // ---- epilogue: lane owns query qn and rows 8*(r/4) + 4*h + r%4 ----
        const uint32_t slot0 = b * 32u;
        uint32_t mw = 0xffffffffu;
        if (a.mask != nullptr) mw = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
        float vs[16];
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            const float4 f = *reinterpret_cast<const float4 *>(a.scales + slot0 + 8 * q4 + 4 * h);
            vs[q4 * 4 + 0] = f.x; vs[q4 * 4 + 1] = f.y; vs[q4 * 4 + 2] = f.z; vs[q4 * 4 + 3] = f.w;
        }
        if (DUMP) {
            if (active) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                    const uint32_t slot = slot0 + i;
                    if (slot < a.n) {
                        const float s = fmaf(float(acc[r]), qs, qb) * vs[r];
                        const size_t o = size_t(qn) * a.n + slot;
                        if (a.acc_out) a.acc_out[o] = acc[r];
                        if (a.score_out) a.score_out[o] = ((mw >> i) & 1u) ? s : __int_as_float(0x7fc00000);
                    }
                }
            }
        } else if (BEST) {
            // A first sampling level without a floor: one candidate per block and query, the best
            // allowed row of the block (a real score of a real row, so the k-th best of these is a
            // floor at least k scanned rows reach, and with rows in no particular order it is the
            // k-th best row of the sample but for the odd pair that shares a block).
            float bs = 0.0f;
            uint32_t bslot = 0xffffffffu;      // none yet
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                const uint32_t slot = slot0 + i;
                const float s = fmaf(float(acc[r]), qs, qb) * vs[r];
                const bool ok = active && slot < a.n && ((mw >> i) & 1u) && s == s;
                if (ok && (bslot == 0xffffffffu || ranks_before(s, slot, bs, bslot))) { bs = s; bslot = slot; }
            }
            const float os_ = __shfl_xor(bs, 32);
            const uint32_t oslot = __shfl_xor(bslot, 32);
            if (oslot != 0xffffffffu && (bslot == 0xffffffffu || ranks_before(os_, oslot, bs, bslot))) { bs = os_; bslot = oslot; }
            if (h == 0 && bslot != 0xffffffffu) {
                const uint32_t pos = atomicAdd(&scnt[qn], 1u);
                if (pos < kSegCap) a.cand[(size_t(qn) * a.seg_stride + vb) * kSegCap + pos] = sort_key(bs, bslot);
            }
        } else if (APPEND) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float s = fmaf(float(acc[r]), qs, qb) * vs[r];
                if (s >= tau_fixed) {
                    const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                    const uint32_t slot = slot0 + i;
                    if (slot < a.n && ((mw >> i) & 1u)) {
                        const uint32_t pos = atomicAdd(&scnt[qn], 1u);
                        if (pos < kSegCap)
                            a.cand[(size_t(qn) * a.seg_stride + vb) * kSegCap + pos] = sort_key(s, slot);
                    }
                }
            }
        } else {
            if (a.share_tau && (j & 3u) == 0u && lane < kQTile) atomicMax(&stau[lane], a.gtau[lane]);
            const float tau = order_unkey(stau[qn]);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                const uint32_t slot = slot0 + i;
                const float s = fmaf(float(acc[r]), qs, qb) * vs[r];
                if (active && s >= tau && (L.cnt < k || ranks_before(s, slot, L.worst_s, L.worst_i))) {
                    if (slot < a.n && ((mw >> i) & 1u)) {
                        if (list_offer(L, ls, li, THREADS, tid, k, s, slot) && a.share_tau) {
                            const int key = order_key(L.worst_s);
                            if (atomicMax(&stau[qn], key) < key) atomicMax(&a.gtau[qn], key);
                        }
                    }
                }
            }
        }
        j = nj_live;
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
    if (APPEND) {
        __syncthreads();
        const int t = tid % kScanThreads;
        if (t < a.nq_tile && vb < vgrid) a.cand_cnt[size_t(t) * a.seg_stride + vb] = scnt[t];
    }
}

// ===========================================================================
// Multi-tile scan, score mode P, append mode only: the weights of NT query
// tiles stay resident in LDS for the whole launch (NT * dim bytes), every wave
// decodes a chunk once and feeds NT tiles' MFMAs from it.  No barrier in the
// main loop.  Used when NT * dim fits the 160 KiB of LDS.
// ===========================================================================

// LB = code bytes of a lane's sixteen that are decoded through the LDS byte table (8: bytes 8..15;
// 4: bytes 12..15, bytes 8..11 then go through the vector ALU like bytes 0..7 and are interleaved
// into the table's (low, high) order by two byte permutes: fewer LDS reads in flight and fewer
// registers, which lets the three-tile instance run four waves per SIMD).
template <int NT, int U, int THREADS, int LB>
__global__ __launch_bounds__(THREADS) void k_scan_p4_multi(ScanArgs a) {
    static_assert(LB == 8 || LB == 4, "table bytes per lane and chunk");
    extern __shared__ __align__(16) uint8_t smem[];
    if (launch_switched_off(a.run_if)) return;
    const int nch = a.nch;
    uint8_t *sW = smem + kDecodeBytes;                             // [NT][nch][2][64 lanes][16], after the byte table
    uint32_t *scnt = reinterpret_cast<uint32_t *>(sW + size_t(NT) * nch * 2048);
    const int tid = threadIdx.x, lane = tid & 63;
    const int qn = lane & 31, h = lane >> 5;
    const int nt_active = (a.nq_tile + kQTile - 1) / kQTile;
    {
        const int live16 = nt_active * nch * 128;
        stage_to_lds<THREADS>(reinterpret_cast<uint4 *>(sW), reinterpret_cast<const uint4 *>(a.tables), live16, tid);
        for (int i = live16 + tid; i < NT * nch * 128; i += THREADS) reinterpret_cast<uint4 *>(sW)[i] = make_uint4(0, 0, 0, 0);
    }
    for (int b = tid; b < 256; b += THREADS) {   // code byte -> (level of its low nibble, level of its high nibble)
        const uint32_t lo = (a.lv[(b & 15) >> 2] >> (8 * (b & 3))) & 0xffu;
        const uint32_t hi = (a.lv[b >> 6] >> (8 * ((b >> 4) & 3))) & 0xffu;
        reinterpret_cast<uint16_t *>(smem)[b] = uint16_t(lo | (hi << 8));
    }
    uint32_t *snext = scnt + NT * kQTile;   // next unclaimed block of this workgroup
    // Per query, in LDS (a block's epilogue reads them; registers are for the stream): scale, bias
    // and floor, and the accumulator bound of k_scan_p4_wide -- a row reaches its query's floor only
    // if its integer sum reaches  floor / (qscale * largest row scale of the block) - qbias / qscale,
    // taken conservatively (1e-5 relative, 2 + 1 absolute), so a tile of a block is scored in
    // floats only when some lane's largest sum is at the bound.  Floors, query scales and biases
    // outside 1e-30 .. 1e30 switch the bound off for that query (every tile scored).
    float4 *s_q = reinterpret_cast<float4 *>(snext + 4);      // [NT * 32] (scale, bias, floor, -)
    float2 *s_b = reinterpret_cast<float2 *>(s_q + NT * kQTile);   // [NT * 32] (ta, tb) of the bound
    float *s_vs = reinterpret_cast<float *>(s_b + NT * kQTile) + (tid >> 6) * 32;   // this wave's: the row scales of the block it finishes, NaN where not allowed
    for (int q = tid; q < NT * kQTile; q += THREADS) {
        scnt[q] = 0u;
        const bool act = q < a.nq_tile;
        const float qs = act ? a.qscale[q] : 0.0f, qb = act ? a.qbias[q] : 0.0f;
        const float tau = act ? order_unkey(a.gtau[q]) : __int_as_float(0x7fc00000);  // NaN: nothing passes
        s_q[q] = make_float4(qs, qb, tau, 0.0f);
        const float inf = __int_as_float(0x7f800000);
        const bool bounded = tau >= 1e-30f && tau <= 1e30f && qs >= 1e-30f && qs <= 1e30f && fabsf(qb) <= 1e30f &&
                             tau / qs < inf;
        const float rb = qb / qs;
        s_b[q] = make_float2(!act ? inf : bounded ? (tau / qs) * (1.0f - 1e-5f) : -inf,
                             act && bounded ? rb + 1e-5f * fabsf(rb) + 2.0f : 0.0f);
    }
    if (tid == 0) *snext = 0u;
    __syncthreads();

    const uint32_t t0 = a.lv[0], t1 = a.lv[1], t2 = a.lv[2], t3 = a.lv[3];
    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;
    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes) + lane;
    const uint32_t w_base = uint32_t(kDecodeBytes + lane * 16), w_tile = uint32_t(nch) * 2048u;

    // Blocks are dealt round-robin to workgroups (logical block m * gridDim.x + blockIdx.x belongs
    // to this one), so neighbouring rows -- clustered data, contiguous allowlists -- spread over
    // all of them; inside a workgroup the waves claim blocks from a shared counter as they go,
    // so all of them finish within one block of each other whatever the SIMD arbitration did.
    // Returns the next block with at least one allowed slot (search.rs:3015-3029), or >= nj.
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

    // The wave's work is one stream of U-chunk groups running through its blocks.  Two register
    // sets take turns: while one group is decoded and multiplied, the next group's codes (of this
    // block, or the head of the next live one) are in flight into the other set, requested as one
    // contiguous burst.  Every group issues the same loads in the same order -- the row scale of
    // its block, then the burst -- so the number of younger loads behind any register is fixed:
    // before chunk u of the current set, 2U - u of them may still be outstanding.
    v16i acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t j = claim();
    int c0 = 0;
    const uint8_t *code_bytes = reinterpret_cast<const uint8_t *>(codes);   // lane offset included

    auto issue = [&](u32x4 (&dst)[U], float &sc, uint32_t jb_phys, int c) {
        load4_async(sc, a.scales + jb_phys * 32u + qn);
        const uint8_t *p = code_bytes + (size_t(jb_phys) * nch + c) * 1024;
        load16_async<0>(dst[0], p);
        if (U > 1) load16_async<1024>(dst[U > 1 ? 1 : 0], p);
        if (U > 2) load16_async<2048>(dst[U > 2 ? 2 : 0], p);
        if (U > 3) load16_async<3072>(dst[U > 3 ? 3 : 0], p);
        static_assert(U <= 4, "immediate offsets cover four chunks");
    };

    auto finish_block = [&](uint32_t b, float my_scale) {
        const uint32_t slot0 = b * 32u;
        uint32_t mw = 0xffffffffu;
        if (a.mask != nullptr) mw = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
        // Rows past the end of the index or outside the allowlist get a NaN scale: their scores
        // then fail the floor compare by themselves, and the per-score path has no other test.
        if (slot0 + 32u > a.n) mw &= (a.n > slot0) ? (0xffffffffu >> (slot0 + 32u - a.n)) : 0u;
        // the block's largest allowed row scale; a negative, huge or non-finite scale (no encoder
        // writes such) or a largest one below 1e-30 switches the bound off for the block
        // (the lane's query number through a move the compiler cannot see through: the addresses of
        // its records are then formed here, per block, instead of living in registers through the stream)
        int qrec = qn;
        asm volatile("v_mov_b32 %0, %0" : "+v"(qrec));
        const bool ok = (mw >> qn) & 1u;
        const bool odd = ok && !(my_scale >= 0.0f && my_scale <= 1e30f);
        // (non-negative floats order like their bit patterns: the maximum on the data-parallel path, no LDS)
        const float vmax = __uint_as_float(wave_umax(ok && !odd ? __float_as_uint(my_scale) : 0u));
        const float inv = 1.0f / vmax;       // all scales zero: +inf, no sum reaches the bound, and every score is zero
        if (lane < 32) s_vs[lane] = ok ? my_scale : __int_as_float(0x7fc00000);   // for the tiles scored below (read by this wave only)
        const bool odd_block = __any(odd) || (vmax > 0.0f && vmax < 1e-30f);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float2 tq = s_b[t * kQTile + qrec];
            const float bf = fmaf(tq.x, inv, -tq.y) - 1.0f;
            int bound;
            asm("v_cvt_i32_f32 %0, %1" : "=v"(bound) : "v"(bf));   // saturates; NaN gives 0
            if (odd_block) bound = int(0x80000000);
            const v16i &c = acc[t];
            int m = max(max(c[0], c[1]), c[2]);       // (one running maximum: the kernel has no register to spare)
            m = max(max(m, c[3]), c[4]);
            m = max(max(m, c[5]), c[6]);
            m = max(max(m, c[7]), c[8]);
            m = max(max(m, c[9]), c[10]);
            m = max(max(m, c[11]), c[12]);
            m = max(max(m, c[13]), c[14]);
            m = max(m, c[15]);
            if (m >= bound) {
                const float4 qp = s_q[t * kQTile + qrec];
                const float *vs = s_vs + 4 * h;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                    const float s = fmaf(float(acc[t][r]), qp.x, qp.y) * vs[8 * (r >> 2) + (r & 3)];
                    if (s >= qp.z) {
                        const int q = t * kQTile + qn;
                        const uint32_t pos = atomicAdd(&scnt[q], 1u);
                        if (pos < kSegCap)
                            a.cand[(size_t(q) * a.seg_stride + blockIdx.x) * kSegCap + pos] = sort_key(s, slot0 + i);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    };

    // One group: request the following group into `nxt`, consume `cur`.  Returns false after the
    // wave's last group (whose request re-reads the current group: a valid address, never used).
    auto phase = [&](u32x4 (&cur)[U], float &cur_sc, u32x4 (&nxt)[U], float &nxt_sc) -> bool {
        const uint32_t b = j * step;
        const bool block_ends = c0 + U >= nch;
        uint32_t pj = j;
        int pc = c0 + U;
        if (block_ends) { pj = claim(); pc = 0; }
        const bool more = pj < nj;
        issue(nxt, nxt_sc, (more ? pj : j) * step, more ? pc : c0);
        // the group's weights: one address per tile, the chunk and the operand as immediate offsets
        uint32_t w_at[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) w_at[t] = w_base + (uint32_t(c0) * 2048u + uint32_t(t) * w_tile);
        static_for<U>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            wait_vm<2 * U - u>(cur[u]);
            // Split decode as in k_scan_p4: code bytes 8..15 of the lane through the byte table
            // (requested first), bytes 0..7 on the vector ALU while those reads and the first
            // operand's weights are on their way; the second operand's weights travel during the
            // first operand's MFMAs.  All LDS traffic of the loop is requested and waited for by
            // hand, so the counts below are exact.
            constexpr int kTab = LB / 2;      // dwords of the second operand that come from the table (two code bytes each)
            uint32_t e[kTab], o[kTab];
            if constexpr (LB == 8) {
                lds_u16(e[0], byte_x2<0>(cur[u].z)); lds_u16(o[0], byte_x2<1>(cur[u].z));
                lds_u16(e[1], byte_x2<2>(cur[u].z)); lds_u16(o[1], byte_x2<3>(cur[u].z));
            }
            lds_u16(e[kTab - 2], byte_x2<0>(cur[u].w)); lds_u16(o[kTab - 2], byte_x2<1>(cur[u].w));
            lds_u16(e[kTab - 1], byte_x2<2>(cur[u].w)); lds_u16(o[kTab - 1], byte_x2<3>(cur[u].w));
            v4i b0[NT], b1[NT];
            static_for<NT>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                lds_b128<u * 2048>(b0[t], w_at[t]);
            });
            const v4i a0 = {int(levels_of(cur[u].x & 0x0f0f0f0fu, t0, t1, t2, t3)),
                            int(levels_of((cur[u].x >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3)),
                            int(levels_of(cur[u].y & 0x0f0f0f0fu, t0, t1, t2, t3)),
                            int(levels_of((cur[u].y >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3))};
            uint32_t z01[2] = {0u, 0u};       // LB = 4: the second operand's first two dwords, from bytes 8..11
            if constexpr (LB == 4) {
                const uint32_t lo = levels_of(cur[u].z & 0x0f0f0f0fu, t0, t1, t2, t3);
                const uint32_t hi = levels_of((cur[u].z >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3);
                z01[0] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);      // (low, high) of byte 8, of byte 9
                z01[1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);      // of bytes 10 and 11
            }
            lds_settle_all(e, o, b0);
            static_for<NT>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                lds_b128<u * 2048 + 1024>(b1[t], w_at[t]);
            });
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0[t], acc[t], 0, 0, 0);
            v4i a1;
            if constexpr (LB == 8) {
                a1 = v4i{int(e[0] | (o[0] << 16)), int(e[1] | (o[1] << 16)), int(e[2] | (o[2] << 16)), int(e[3] | (o[3] << 16))};
            } else {
                a1 = v4i{int(z01[0]), int(z01[1]), int(e[0] | (o[0] << 16)), int(e[1] | (o[1] << 16))};
            }
            lds_settle_all(e, o, b1);
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1[t], acc[t], 0, 0, 0);
        });
        if (block_ends) {
            wait_vm<U + 1>(cur_sc);   // this group's own scale: only the request issued above is younger
            finish_block(b, cur_sc);
        }
        j = pj;
        c0 = pc;
        return more;
    };

    if (j < nj) {
        u32x4 bufA[U], bufB[U];
        float scA, scB;
        issue(bufA, scA, j * step, 0);
        while (phase(bufA, scA, bufB, scB) && phase(bufB, scB, bufA, scA)) {}
        asm volatile("s_waitcnt vmcnt(0)");
    }
    __syncthreads();
    for (int q = tid; q < a.nq_tile; q += THREADS) a.cand_cnt[size_t(q) * a.seg_stride + blockIdx.x] = scnt[q];
}

// ===========================================================================
// Batched scan, score mode P, append mode only: one pass serves NT query tiles
// (NT*32 queries).  A workgroup walks groups of 4*MW blocks; each wave decodes
// its MW blocks once per chunk and feeds NT tiles' MFMAs from the same decoded
// operand, so the nibble decode -- the VALU cost that bounds the single-tile
// kernel -- is amortised NT times.  The NT tiles' weights (NT * dim bytes) do
// not fit LDS whole, so they stream through it in slices of KC chunks, double
// buffered, shared by the four waves and re-read from L2 once per block group.
// ===========================================================================

template <int NT, int MW, int KC, int OCC>
__global__ __launch_bounds__(kScanThreads, OCC) void k_scan_p4_batched(ScanArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    if (launch_switched_off(a.run_if)) return;
    constexpr int kSliceBytes = NT * KC * 2048;           // one slice of all tiles
    constexpr int kStage = kSliceBytes / (kScanThreads * 16);  // uint4 per thread per slice
    static_assert(kSliceBytes % (kScanThreads * 16) == 0, "slice must split evenly over the workgroup");
    uint8_t *sB = smem;                                   // [2][NT][KC][2][1024]
    uint32_t *scnt = reinterpret_cast<uint32_t *>(smem + 2 * kSliceBytes);  // [NT*32]
    const int nch = a.nch;
    const int nslices = nch / KC;                         // host guarantees nch % KC == 0
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qn = lane & 31, h = lane >> 5;
    const int nt_active = (a.nq_tile + kQTile - 1) / kQTile;
    const uint32_t t0 = a.lv[0], t1 = a.lv[1], t2 = a.lv[2], t3 = a.lv[3];

    for (int i = tid; i < NT * kQTile; i += kScanThreads) scnt[i] = 0u;

    float qs[NT], qb[NT], tau[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int q = t * kQTile + qn;
        const bool act = q < a.nq_tile;
        qs[t] = act ? a.qscale[q] : 0.0f;
        qb[t] = act ? a.qbias[q] : 0.0f;
        tau[t] = act ? order_unkey(a.gtau[q]) : __int_as_float(0x7fc00000);  // NaN: nothing passes
    }

    const uint32_t step = a.b_step;
    const uint32_t nj = (a.n_blocks + step - 1) / step;   // logical blocks
    constexpr uint32_t kGroup = 4 * MW;                   // logical blocks per workgroup iteration
    const uint32_t ngroups = (nj + kGroup - 1) / kGroup;

    // staging of weight slices: thread copies kStage uint4 per slice; slice s of tile t lives at
    // tables + t*nch*2048 + s*KC*2048 (KC*2048 contiguous bytes)
    uint4 stage[kStage];
    auto load_slice = [&](int sl) {
#pragma unroll
        for (int e = 0; e < kStage; ++e) {
            const int idx = e * kScanThreads + tid;               // uint4 index within the slice
            const int t = idx / (KC * 128), r = idx % (KC * 128);
            if (t < nt_active)
                stage[e] = reinterpret_cast<const uint4 *>(a.tables + (size_t(t) * nch + size_t(sl) * KC) * 2048)[r];
            else
                stage[e] = make_uint4(0, 0, 0, 0);
        }
    };
    auto store_slice = [&](int buf) {
        uint4 *dst = reinterpret_cast<uint4 *>(sB + buf * kSliceBytes);
#pragma unroll
        for (int e = 0; e < kStage; ++e) dst[e * kScanThreads + tid] = stage[e];
    };

    const uint4 *codes = reinterpret_cast<const uint4 *>(a.codes) + lane;
    uint32_t g = blockIdx.x;
    if (g >= ngroups) {                                   // whole workgroup leaves together, with empty segments
        for (int q = tid; q < a.nq_tile; q += kScanThreads) a.cand_cnt[size_t(q) * a.seg_stride + blockIdx.x] = 0u;
        return;
    }
    load_slice(0);
    store_slice(0);
    __syncthreads();
    int ring = 0;                                         // buffer holding the slice about to be consumed

    for (; g < ngroups; g += gridDim.x) {
        // this wave's MW logical blocks
        uint32_t jb[MW];
        bool live[MW];
        uint32_t mw[MW];
#pragma unroll
        for (int m = 0; m < MW; ++m) {
            jb[m] = g * kGroup + wave * MW + m;
            live[m] = jb[m] < nj;
            mw[m] = 0xffffffffu;
            if (live[m] && a.mask != nullptr) {
                const uint32_t b = jb[m] * step;
                mw[m] = uint32_t(a.mask[b >> 1] >> ((b & 1) * 32));
                live[m] = mw[m] != 0u;                    // block skip (search.rs:3015-3029)
            }
        }
        v16i acc[MW][NT];
#pragma unroll
        for (int m = 0; m < MW; ++m)
#pragma unroll
            for (int t = 0; t < NT; ++t) acc[m][t] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

        uint4 abuf[MW][KC];                               // codes of the slice being computed
#pragma unroll
        for (int m = 0; m < MW; ++m)
#pragma unroll
            for (int c = 0; c < KC; ++c)
                abuf[m][c] = live[m] ? load_stream16(&codes[(size_t(jb[m]) * step * nch + c) * 64]) : make_uint4(0, 0, 0, 0);

        for (int sl = 0; sl < nslices; ++sl) {
            const bool more = sl + 1 < nslices || g + gridDim.x < ngroups;
            const int next_sl = sl + 1 < nslices ? sl + 1 : 0;
            if (more) load_slice(next_sl);
            uint4 acur[MW][KC];
#pragma unroll
            for (int m = 0; m < MW; ++m)
#pragma unroll
                for (int c = 0; c < KC; ++c) acur[m][c] = abuf[m][c];
            if (sl + 1 < nslices) {
#pragma unroll
                for (int m = 0; m < MW; ++m)
#pragma unroll
                    for (int c = 0; c < KC; ++c)
                        abuf[m][c] = live[m] ? load_stream16(&codes[(size_t(jb[m]) * step * nch + (sl + 1) * KC + c) * 64])
                                             : make_uint4(0, 0, 0, 0);
            }
            const uint4 *bl = reinterpret_cast<const uint4 *>(sB + ring * kSliceBytes) + lane;
#pragma unroll
            for (int c = 0; c < KC; ++c) {
                v4i alo[MW], ahi[MW];
#pragma unroll
                for (int m = 0; m < MW; ++m) {
                    const uint32_t x[4] = {acur[m][c].x, acur[m][c].y, acur[m][c].z, acur[m][c].w};
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        alo[m][d] = int(levels_of(x[d] & 0x0f0f0f0fu, t0, t1, t2, t3));
                        ahi[m][d] = int(levels_of((x[d] >> 4) & 0x0f0f0f0fu, t0, t1, t2, t3));
                    }
                }
                // all low-nibble products first, then all high-nibble ones: the two MFMAs that
                // chain on one accumulator end up NT*MW instructions apart instead of back to back
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const uint4 wl = bl[((t * KC + c) * 2) * 64];
                    const v4i blo = {int(wl.x), int(wl.y), int(wl.z), int(wl.w)};
#pragma unroll
                    for (int m = 0; m < MW; ++m)
                        acc[m][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(alo[m], blo, acc[m][t], 0, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const uint4 wh = bl[((t * KC + c) * 2 + 1) * 64];
                    const v4i bhi = {int(wh.x), int(wh.y), int(wh.z), int(wh.w)};
#pragma unroll
                    for (int m = 0; m < MW; ++m)
                        acc[m][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ahi[m], bhi, acc[m][t], 0, 0, 0);
                }
            }
            if (more) store_slice(ring ^ 1);
            __syncthreads();
            ring ^= 1;
        }

        // ---- epilogue ----
#pragma unroll
        for (int m = 0; m < MW; ++m) {
            if (!live[m]) continue;
            const uint32_t slot0 = jb[m] * step * 32u;
            float vs[16];
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const float4 f = *reinterpret_cast<const float4 *>(a.scales + slot0 + 8 * q4 + 4 * h);
                vs[q4 * 4 + 0] = f.x; vs[q4 * 4 + 1] = f.y; vs[q4 * 4 + 2] = f.z; vs[q4 * 4 + 3] = f.w;
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float s = fmaf(float(acc[m][t][r]), qs[t], qb[t]) * vs[r];
                    if (s >= tau[t]) {
                        const int i = 8 * (r >> 2) + 4 * h + (r & 3);
                        const uint32_t slot = slot0 + i;
                        if (slot < a.n && ((mw[m] >> i) & 1u)) {
                            const int q = t * kQTile + qn;
                            const uint32_t pos = atomicAdd(&scnt[q], 1u);
                            if (pos < kSegCap)
                                a.cand[(size_t(q) * a.seg_stride + blockIdx.x) * kSegCap + pos] = sort_key(s, slot);
                        }
                    }
                }
            }
        }
    }
    __syncthreads();
    for (int q = tid; q < a.nq_tile; q += kScanThreads) a.cand_cnt[size_t(q) * a.seg_stride + blockIdx.x] = scnt[q];
}

// ===========================================================================
// Final merge of the per-lane lists of one query tile.
// One workgroup per query: every thread folds a strided subset of the lists
// into a private top-k, then the 256*k survivors are bitonic-sorted.
// ===========================================================================

__global__ __launch_bounds__(256) void k_merge(const float *__restrict__ part_scores,
                                               const uint32_t *__restrict__ part_idx,
                                               const int *__restrict__ part_cnt, int total_threads, int qmod,
                                               int k, int k_eff, int sort_n, float *__restrict__ out_scores,
                                               int64_t *__restrict__ out_idx, int *__restrict__ out_tau) {
    extern __shared__ __align__(16) uint8_t msm[];
    float *ls = reinterpret_cast<float *>(msm);
    uint32_t *li = reinterpret_cast<uint32_t *>(ls + k * 256);
    uint64_t *keys = reinterpret_cast<uint64_t *>(li + k * 256);
    __shared__ int total;
    const int qn = blockIdx.x;
    const int t = threadIdx.x;
    if (t == 0) total = 0;
    LaneList L{0, 0.0f, 0u, 0};
    // lane (gt % 64) of every wave owns query (gt % 64) % qmod
    const int per_wave = 64 / qmod;
    const int n_lists = total_threads / 64 * per_wave;
    for (int l = t; l < n_lists; l += 256) {
        const int gt = (l / per_wave) * 64 + (l % per_wave) * qmod + qn;
        const int cnt = part_cnt[gt];
        for (int e = 0; e < cnt; ++e)
            list_offer(L, ls, li, 256, t, k, part_scores[size_t(e) * total_threads + gt],
                       part_idx[size_t(e) * total_threads + gt]);
    }
    __syncthreads();
    const int base = atomicAdd(&total, L.cnt);
    for (int e = 0; e < L.cnt; ++e) keys[base + e] = sort_key(ls[e * 256 + t], li[e * 256 + t]);
    __syncthreads();
    for (int i = total + t; i < sort_n; i += 256) keys[i] = 0;  // below every real key
    __syncthreads();
    for (int size = 2; size <= sort_n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int i = t; i < sort_n / 2; i += 256) {
                const int lo = 2 * i - (i & (stride - 1));
                const int hi = lo + stride;
                const bool desc = (lo & size) == 0;
                const uint64_t x = keys[lo], y = keys[hi];
                if ((x < y) == desc) { keys[lo] = y; keys[hi] = x; }
            }
            __syncthreads();
        }
    }
    if (out_tau != nullptr) {
        // sampling pass: publish a floor that at least k_eff scanned slots reach
        if (t == 0) {
            float s = 0.0f; uint32_t idx = 0;
            if (total >= k_eff && k_eff <= sort_n) sort_unkey(keys[k_eff - 1], s, idx);
            out_tau[qn] = (total >= k_eff && k_eff <= sort_n) ? order_key(s == 0.0f ? -0.0f : s) : kTauInit;
        }
        return;
    }
    for (int j = t; j < k_eff; j += 256) {
        float s; uint32_t idx;
        sort_unkey(keys[j], s, idx);
        out_scores[size_t(qn) * k_eff + j] = s;
        out_idx[size_t(qn) * k_eff + j] = int64_t(idx);
    }
}

// ===========================================================================
// Final selection over the candidates an append-mode scan collected: one
// workgroup per query sorts its (few) candidate keys in LDS and emits the first
// k_eff.  A query whose candidates did not fit is flagged for the caller to
// redo through the list path.
// ===========================================================================

__device__ __forceinline__ uint64_t wave_umax64(uint64_t v) {
    const uint32_t hi = uint32_t(v >> 32), lo = uint32_t(v);
    const uint32_t mhi = wave_umax(hi);
    const uint32_t mlo = wave_umax(hi == mhi ? lo : 0u);
    return (uint64_t(mhi) << 32) | mlo;
}
// Eight keys in descending order (Batcher's odd-even merge network, 19 exchanges).
__device__ __forceinline__ void sort8_desc(uint64_t (&r)[8]) {
    auto ce = [&](int i, int j) { if (r[i] < r[j]) { const uint64_t x = r[i]; r[i] = r[j]; r[j] = x; } };
    ce(0, 1); ce(2, 3); ce(4, 5); ce(6, 7);
    ce(0, 2); ce(1, 3); ce(4, 6); ce(5, 7);
    ce(1, 2); ce(5, 6);
    ce(0, 4); ce(1, 5); ce(2, 6); ce(3, 7);
    ce(2, 4); ce(3, 5);
    ce(1, 2); ce(3, 4); ce(5, 6);
}
// Sixteen keys in descending order: two sorted eights, then a bitonic merge (70 exchanges).
__device__ __forceinline__ void sort16_desc(uint64_t (&r)[16]) {
    auto ce = [&](int i, int j) { if (r[i] < r[j]) { const uint64_t x = r[i]; r[i] = r[j]; r[j] = x; } };
    uint64_t a[8], b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { a[e] = r[e]; b[e] = r[8 + e]; }
    sort8_desc(a);
    sort8_desc(b);
#pragma unroll
    for (int e = 0; e < 8; ++e) { r[e] = a[e]; r[8 + e] = b[e]; }
#pragma unroll
    for (int i = 0; i < 8; ++i) ce(i, 15 - i);              // the eight larger in front, both halves bitonic
#pragma unroll
    for (int stride = 4; stride >= 1; stride >>= 1) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            if ((i & stride) == 0) ce(i, i + stride);
    }
}
// The `need` (<= 32) largest of the wave's keys -- N per lane, sorted descending, 0 = none,
// non-zero keys distinct -- in order: lane i returns the i-th largest (0 beyond what there is).
// One largest key is found and retired per turn; nothing touches LDS.
template <int N>
__device__ __forceinline__ uint64_t wave_top(uint64_t (&r)[N], uint32_t need, uint32_t lane) {
    uint64_t mine = 0ull;
    for (uint32_t it = 0; it < need; ++it) {
        const uint64_t m = wave_umax64(r[0]);
        if (lane == it) mine = m;
        if (r[0] == m && m != 0ull) {
#pragma unroll
            for (int e = 0; e < N - 1; ++e) r[e] = r[e + 1];
            r[N - 1] = 0ull;
        }
    }
    return mine;
}

constexpr int kFinalThreads = 1024;
constexpr int kFinalLong = kFinalCap / 8;   // segments of more than 8 keys that fit the sort buffer

__global__ __launch_bounds__(kFinalThreads) void k_final(const uint64_t *__restrict__ cand,
                                               const uint32_t *__restrict__ cand_cnt, uint32_t n_seg,
                                               uint32_t seg_stride, int k_eff, int k_floor,
                                               float *__restrict__ out_scores, int64_t *__restrict__ out_idx,
                                               uint32_t *__restrict__ overflow, int *__restrict__ tau_out,
                                               int tau_stride_q, int keep_floor, int *__restrict__ raise_out,
                                               const uint32_t *__restrict__ row_map, uint32_t *level_over,
                                               uint32_t *clear_flag, const uint32_t *run_if) {
    __shared__ uint64_t keys[kFinalCap];
    __shared__ uint32_t wave_sum[kFinalThreads / 64];
    __shared__ uint32_t any_full, long_n, any_long, any_over8;
    __shared__ uint32_t long_seg[kFinalLong], long_pos[kFinalLong], long_cnt[kFinalLong];
    const int qn = blockIdx.x;
    const int t = threadIdx.x;
    const bool sampling = tau_out != nullptr;
    int *tau_slot = sampling ? tau_out + (qn / tau_stride_q) * kQTile + qn % tau_stride_q : nullptr;
    if (launch_switched_off(run_if)) return;
    if (clear_flag != nullptr && qn == 0 && t == 0) *clear_flag = 0u;
    if (t == 0) { any_full = 0u; long_n = 0u; any_long = 0u; any_over8 = 0u; }
    __syncthreads();
    // every thread owns a contiguous run of this query's segments
    const uint32_t per = (n_seg + kFinalThreads - 1) / kFinalThreads;
    const uint32_t s0 = min(uint32_t(t) * per, n_seg), s1 = min(s0 + per, n_seg);
    const uint32_t *cnt = cand_cnt + size_t(qn) * seg_stride;
    constexpr uint32_t kShort = 16;
    // One segment per thread (the usual case): its head is requested together with its count, not
    // after it -- the segment's memory is there whatever the count says -- which takes one trip to
    // memory out of a kernel that is nothing but latency.
    const bool one_each = per == 1;
    uint64_t head[kShort];
#pragma unroll
    for (uint32_t e = 0; e < kShort; ++e) head[e] = 0ull;
    uint32_t mine = 0;
    if (one_each) {
        if (s0 < s1) {
            const uint64_t *src = cand + (size_t(qn) * seg_stride + s0) * kSegCap;
            const uint32_t c = cnt[s0];
#pragma unroll
            for (uint32_t e = 0; e < kShort; ++e) head[e] = src[e];
            if (c > kSegCap) any_full = 1u;
            mine = min(c, uint32_t(kSegCap));
            if (mine > kShort) any_long = 1u;
            if (mine > 8u) any_over8 = 1u;
        }
    } else {
        for (uint32_t sg = s0; sg < s1; ++sg) {
            const uint32_t c = cnt[sg];
            if (c > kSegCap) any_full = 1u;
            mine += min(c, uint32_t(kSegCap));
        }
    }
    // exclusive prefix over the 256 threads
    uint32_t incl = mine;
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t v = __shfl_up(incl, off);
        if ((t & 63) >= off) incl += v;
    }
    if ((t & 63) == 63) wave_sum[t >> 6] = incl;
    __syncthreads();
    uint32_t base = incl - mine, total = 0;
    for (int w = 0; w < kFinalThreads / 64; ++w) { if (w < (t >> 6)) base += wave_sum[w]; total += wave_sum[w]; }
    const bool too_many = total > uint32_t(kFinalCap);
    // A sampling level whose candidates did not all fit yields its floor from the subset that was
    // kept: a valid floor, but possibly far below the k_floor-th best of the level.  The flag lets
    // the caller's conditional launches repeat the level from that floor, which then fits.
    if (sampling && level_over != nullptr && t == 0 && (too_many || any_full)) *level_over = 1u;
    // A final pass whose candidates did not fit: flag 1 = the caller repeats the full scan for this
    // query with the raised floor written below (the k_floor-th best of what was kept -- real
    // slots, so a valid lower bound of the true k-th best, and above the floor that let too many
    // through); flag 2 = straight to the exact path (no such floor: fewer than k_eff candidates,
    // or the caller takes no raised floors).
    bool raising = false;
    if (!sampling) {
        const bool redo = too_many || any_full || total < uint32_t(k_eff);
        raising = redo && raise_out != nullptr && total >= uint32_t(k_eff);
        if (t == 0) overflow[qn] = redo ? (raising ? 1u : 2u) : 0u;
        if (redo && !raising) return;
    }
    if (sampling && total < uint32_t(k_eff)) {
        // Too few allowed slots reached the floor in this sample.  The floor of the level before
        // (k_floor scanned slots reach it) is still a valid lower bound: it stays.  Only the
        // first level, which reads the standing array of open floors, has none to keep.
        if (t == 0 && !keep_floor) *tau_slot = kTauInit;
        return;
    }
    const uint32_t c_all = min(total, uint32_t(kFinalCap));
    const uint32_t need = (sampling || raising) ? min(uint32_t(k_floor), c_all) : uint32_t(k_eff);   // leading keys wanted, in order
    // Few keys wanted and every thread already holds its whole segment in registers (the usual
    // single-query case: some thousand candidates, a few per workgroup of the scan): no gather, no
    // sort.  Every wave picks its `need` largest by rounds of wave-wide maxima, the 16 x 32 picks
    // meet in LDS, and the first wave picks the `need` largest of those the same way.
    const bool in_registers = one_each && any_long == 0u && need <= 32u;
    if (in_registers) {
        const uint32_t lane = uint32_t(t) & 63u, wv = uint32_t(t) >> 6;
#pragma unroll
        for (uint32_t e = 0; e < kShort; ++e) if (e >= mine) head[e] = 0ull;
        uint64_t pick;
        if (any_over8 == 0u) {          // the usual case: eight keys per thread at most
            uint64_t r8[8];
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) r8[e] = head[e];
            sort8_desc(r8);
            pick = wave_top(r8, need, lane);
        } else {
            sort16_desc(head);
            pick = wave_top(head, need, lane);
        }
        if (lane < 32u) keys[wv * 32u + lane] = pick;
        __syncthreads();
        if (wv == 0) {
            uint64_t r[8];
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) r[e] = keys[lane * 8u + e];
            sort8_desc(r);
            const uint64_t best = wave_top(r, need, lane);
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            if (lane < 32u) keys[lane] = best;
        }
        __syncthreads();
    } else {
    // gather (a sampling level may keep any subset: dropping what does not fit only loosens the floor).
    // A thread copies a short segment itself, its loads in flight together; long ones (the first
    // sampling level fills a few segments to the brim) go on a list the waves then share, four
    // segments per wave and turn, a key per lane.
    uint32_t pos = base;
    for (uint32_t sg = s0; sg < s1; ++sg) {
        const uint32_t c = one_each ? mine : min(cnt[sg], uint32_t(kSegCap));
        const uint64_t *src = cand + (size_t(qn) * seg_stride + sg) * kSegCap;
        if (c <= kShort) {
            uint64_t v[kShort];
#pragma unroll
            for (uint32_t e = 0; e < kShort; ++e) v[e] = one_each ? head[e] : (e < c ? src[e] : 0ull);
#pragma unroll
            for (uint32_t e = 0; e < kShort; ++e)
                if (e < c && pos + e < uint32_t(kFinalCap)) keys[pos + e] = v[e];
        } else {
            const uint32_t slot = atomicAdd(&long_n, 1u);
            if (slot < uint32_t(kFinalLong)) {
                long_seg[slot] = sg;
                long_pos[slot] = pos;
                long_cnt[slot] = c;
            } else {                      // more long segments than the list holds: copy in place
                for (uint32_t e = 0; e < c; ++e)
                    if (pos + e < uint32_t(kFinalCap)) keys[pos + e] = src[e];
            }
        }
        pos += c;
    }
    __syncthreads();
    const uint32_t n_long = min(long_n, uint32_t(kFinalLong));
    constexpr uint32_t kWavesF = kFinalThreads / 64;
    for (uint32_t i0 = uint32_t(t >> 6); i0 < n_long; i0 += kWavesF * 4) {   // four segments' loads in flight per wave
        uint64_t v[4];
        uint32_t at[4];
        bool ok[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t i = i0 + u * kWavesF;
            ok[u] = false;
            at[u] = 0;
            v[u] = 0ull;
            if (i < n_long) {
                at[u] = long_pos[i] + uint32_t(t & 63);
                ok[u] = uint32_t(t & 63) < long_cnt[i] && at[u] < uint32_t(kFinalCap);
                if (ok[u]) v[u] = cand[(size_t(qn) * seg_stride + long_seg[i]) * kSegCap + (t & 63)];
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
            if (ok[u]) keys[at[u]] = v[u];
    }
    // leading keys kept in order by the per-wave sorts and merges below (a power of two >= need), or 0: full sort
    const uint32_t keep = need <= 64u ? 64u : need <= 128u ? 128u : need <= 256u ? 256u : 0u;
    uint32_t sort_n = keep ? keep : 2u;
    while (sort_n < c_all) sort_n <<= 1;
    __syncthreads();
    for (uint32_t i = c_all + t; i < sort_n; i += kFinalThreads) keys[i] = 0ull;
    __syncthreads();
    if (keep != 0u) {
        // Few keys wanted: every wave sorts a chunk of its own, no barrier inside (LDS serves a
        // wave's requests in order), and a tree of merges -- the `keep` larger of two sorted runs
        // of `keep` form a bitonic run, log2(keep) strides sort it -- leaves the `keep` best of all
        // in front.
        const uint32_t lane = uint32_t(t) & 63u, wv = uint32_t(t) >> 6;
        const uint32_t len = max(keep, sort_n / (kFinalThreads / 64));
        const uint32_t n_chunks = sort_n / len;
        auto wave_sync = []() {
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        };
        auto swap_down = [&](uint32_t lo, uint32_t hi) {   // larger key to the lower index
            const uint64_t x = keys[lo], y = keys[hi];
            if (x < y) { keys[lo] = y; keys[hi] = x; }
        };
        if (wv < n_chunks) {
            const uint32_t at = wv * len;
            for (uint32_t size = 2; size <= len; size <<= 1) {
                for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
                    for (uint32_t i = lane; i < len / 2; i += 64) {
                        const uint32_t lo = 2 * i - (i & (stride - 1));
                        const uint32_t hi = lo + stride;
                        if ((lo & size) == 0) swap_down(at + lo, at + hi);
                        else swap_down(at + hi, at + lo);
                    }
                    wave_sync();
                }
            }
        }
        for (uint32_t step = 1; step < n_chunks; step <<= 1) {
            __syncthreads();
            if (wv % (2 * step) == 0 && wv + step < n_chunks) {
                const uint32_t at = wv * len, other = (wv + step) * len;
                for (uint32_t i = lane; i < keep; i += 64) {
                    const uint64_t x = keys[at + i], y = keys[other + keep - 1u - i];
                    if (x < y) keys[at + i] = y;
                }
                wave_sync();
                for (uint32_t stride = keep / 2; stride > 0; stride >>= 1) {
                    for (uint32_t i = lane; i < keep / 2; i += 64) {
                        const uint32_t lo = 2 * i - (i & (stride - 1));
                        swap_down(at + lo, at + lo + stride);
                    }
                    wave_sync();
                }
            }
        }
        __syncthreads();
    } else {
        for (uint32_t size = 2; size <= sort_n; size <<= 1) {
            for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
                for (uint32_t i = t; i < sort_n / 2; i += kFinalThreads) {
                    const uint32_t lo = 2 * i - (i & (stride - 1));
                    const uint32_t hi = lo + stride;
                    const bool desc = (lo & size) == 0;
                    const uint64_t x = keys[lo], y = keys[hi];
                    if ((x < y) == desc) { keys[lo] = y; keys[hi] = x; }
                }
                __syncthreads();
            }
        }
    }
    }   // gather and sort through LDS
    if (sampling || raising) {
        if (t == 0) {
            // the floor: the k_floor-th best sampled score (k_floor >= k_eff steadies the estimate)
            const uint32_t pick = min(uint32_t(k_floor), c_all) - 1;
            float s; uint32_t idx;
            sort_unkey(keys[pick], s, idx);
            *(sampling ? tau_slot : raise_out + qn) = order_key(s == 0.0f ? -0.0f : s);
        }
        return;
    }
    const size_t row = row_map ? size_t(row_map[qn]) : size_t(qn);   // a repeated pass writes to the rows of the queries it repeats
    for (int jj = t; jj < k_eff; jj += kFinalThreads) {
        float s; uint32_t idx;
        sort_unkey(keys[jj], s, idx);
        out_scores[row * k_eff + jj] = s;
        out_idx[row * k_eff + jj] = int64_t(idx);
    }
}

// ===========================================================================
// Bandwidth probes: a pure read (sum) and a plain copy over a caller buffer.
// They calibrate what the scan can hope for on this device and give the
// hardware counters a kernel of known traffic to be scaled against.
// ===========================================================================

// The read probe uses the pattern that reads fastest on this device: every wave takes whole
// 8 KiB runs (eight 16-byte loads per lane in flight), with the non-temporal hint.
__global__ __launch_bounds__(256) void k_probe_read(const uint4 *__restrict__ src, size_t n16, uint32_t *sink) {
    uint32_t acc = 0;
    const size_t wave = (size_t(blockIdx.x) * 256 + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    const size_t n_waves = size_t(gridDim.x) * 4;
    constexpr size_t kRun = 64 * 8;   // 16-byte words per run
    size_t r = wave;
    for (; (r + 1) * kRun <= n16; r += n_waves) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load_stream16(src + r * kRun + u * 64 + lane);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    // the words behind the last whole run
    const size_t done = (n16 / kRun) * kRun;
    for (size_t i = done + size_t(blockIdx.x) * 256 + threadIdx.x; i < n16; i += size_t(gridDim.x) * 256) {
        const uint4 a = src[i];
        acc += a.x ^ a.y ^ a.z ^ a.w;
    }
    if (acc == 0x12345678u) *sink = acc;  // keeps the loads alive; practically never taken
}

__global__ __launch_bounds__(256) void k_probe_copy(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
    size_t i = size_t(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = size_t(gridDim.x) * 256;
    for (; i < n16; i += stride) dst[i] = src[i];
}

hipError_t launch_probe(const void *src, void *dst, size_t bytes, int copy, uint32_t *sink, hipStream_t s) {
    const size_t n16 = bytes / 16;
    if (copy) hipLaunchKernelGGL(k_probe_copy, dim3(256 * 8), dim3(256), 0, s, static_cast<const uint4 *>(src),
                                 static_cast<uint4 *>(dst), n16);
    else hipLaunchKernelGGL(k_probe_read, dim3(256 * 8), dim3(256), 0, s, static_cast<const uint4 *>(src), n16, sink);
    return hipGetLastError();
}

// ===========================================================================
// Launchers
// ===========================================================================

hipError_t launch_seq_to_native(const uint8_t *d_seq, uint8_t *d_native, const Geometry &g, size_t first_block,
                                size_t n_blocks, hipStream_t s) {
    if (n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_seq_to_native, dim3(unsigned(n_blocks * g.nch)), dim3(256), 0, s, d_seq, d_native, g.G,
                       g.nch, first_block);
    return hipGetLastError();
}

hipError_t launch_native_to_seq(const uint8_t *d_native, uint8_t *d_seq, const Geometry &g, size_t first_block,
                                size_t n_blocks, hipStream_t s) {
    if (n_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_native_to_seq, dim3(unsigned(n_blocks * g.nch)), dim3(256), 0, s, d_native, d_seq, g.G,
                       g.nch, first_block);
    return hipGetLastError();
}

hipError_t launch_append_rows(const uint8_t *d_rows, uint8_t *d_native, const Geometry &g, size_t old_n,
                              size_t n_new, hipStream_t s) {
    const size_t total = n_new * size_t(g.G);
    if (total == 0) return hipSuccess;
    hipLaunchKernelGGL(k_append_rows, dim3(unsigned((total + 255) / 256)), dim3(256), 0, s, d_rows, d_native, g.G,
                       g.nch, old_n, n_new);
    return hipGetLastError();
}

hipError_t launch_move_lane(uint8_t *d_native, float *d_scales, const Geometry &g, size_t src, size_t dst,
                            hipStream_t s) {
    hipLaunchKernelGGL(k_move_lane, dim3(unsigned((g.G + 255) / 256)), dim3(256), 0, s, d_native, d_scales, g.G,
                       g.nch, src, dst);
    return hipGetLastError();
}

hipError_t launch_gather_redo(const float *d_q, const uint32_t *d_rows, const int *d_raised, int dim, int tile_q,
                              size_t n_redo, float *d_q_out, int *d_tau_out, hipStream_t s) {
    if (n_redo == 0) return hipSuccess;
    hipLaunchKernelGGL(k_gather_redo, dim3(unsigned(n_redo)), dim3(256), 0, s, d_q, d_rows, d_raised, dim, tile_q,
                       d_q_out, d_tau_out);
    return hipGetLastError();
}

hipError_t launch_fill_i32(int *p, int v, size_t n, hipStream_t s) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(k_fill_i32, dim3(unsigned((n + 255) / 256)), dim3(256), 0, s, p, v, n);
    return hipGetLastError();
}

template <typename K>
static hipError_t allow_lds(K kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               int(bytes));
}

hipError_t launch_rotate(const float *d_q, float *d_out, const float *d_signs, const uint32_t *d_perms, int dim,
                         int block, float inv_sqrt_block, size_t nq, hipStream_t s) {
    if (nq == 0) return hipSuccess;
    const size_t lds = size_t(2) * dim * sizeof(float);
    hipError_t e = allow_lds(k_rotate, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(k_rotate, dim3(unsigned(nq)), dim3(256), lds, s, d_q, d_out, d_signs, d_perms, dim, block,
                       inv_sqrt_block);
    return hipGetLastError();
}

hipError_t launch_calibrate(const float *d_qrot, float *d_qcal, float *d_bias_corr, const float *d_shift,
                            const float *d_scale, int dim, size_t nq, hipStream_t s) {
    if (nq == 0) return hipSuccess;
    hipLaunchKernelGGL(k_calibrate, dim3(unsigned(nq)), dim3(256), 0, s, d_qrot, d_qcal, d_bias_corr, d_shift,
                       d_scale, dim);
    return hipGetLastError();
}

hipError_t launch_build_p(const float *d_qcal, const float *d_bias_corr, uint8_t *d_wfrag, float *d_qscale,
                          float *d_qbias, int dim, int G, int nch, float cs, size_t nq, size_t nq_padded,
                          bool split, hipStream_t s) {
    if (nq_padded == 0) return hipSuccess;
    hipLaunchKernelGGL(k_build_p, dim3(unsigned(nq_padded)), dim3(256), 0, s, d_qcal, d_bias_corr, d_wfrag, d_qscale,
                       d_qbias, dim, G, nch, cs, nq, split);
    return hipGetLastError();
}

hipError_t launch_prep_p(const float *d_q, const float *d_signs, const uint32_t *d_perms, int dim, int block,
                         float inv_sqrt_block, const float *d_shift, const float *d_scale, uint8_t *d_wfrag,
                         float *d_qscale, float *d_qbias, int G, int nch, float cs, size_t nq, size_t nq_padded, bool split,
                         hipStream_t s) {
    if (nq_padded == 0) return hipSuccess;
    const size_t lds = size_t(2) * dim * sizeof(float);
    hipError_t e = allow_lds(k_prep_p, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(k_prep_p, dim3(unsigned(nq_padded)), dim3(256), lds, s, d_q, d_signs, d_perms, dim, block,
                       inv_sqrt_block, d_shift, d_scale, d_wfrag, d_qscale, d_qbias, G, nch, cs, nq, split);
    return hipGetLastError();
}

hipError_t launch_build_lut(const float *d_qcal, const float *d_bias_corr, const float *d_centroids, uint8_t *d_lut,
                            float *d_qscale, float *d_qbias, int dim, int bits, int G, int nch, size_t nq,
                            size_t nq_padded, hipStream_t s) {
    if (nq_padded == 0) return hipSuccess;
    const size_t lds = size_t(2) * G * sizeof(float);
    hipError_t e = hipSuccess;
#define TV_LAUNCH_LUT(B)                                                                                         \
    e = allow_lds(k_build_lut<B>, lds);                                                                          \
    if (e != hipSuccess) return e;                                                                               \
    hipLaunchKernelGGL(k_build_lut<B>, dim3(unsigned(nq_padded)), dim3(256), lds, s, d_qcal, d_bias_corr,        \
                       d_centroids, d_lut, d_qscale, d_qbias, dim, G, nch, nq)
    if (bits == 2) { TV_LAUNCH_LUT(2); }
    else if (bits == 3) { TV_LAUNCH_LUT(3); }
    else { TV_LAUNCH_LUT(4); }
#undef TV_LAUNCH_LUT
    return hipGetLastError();
}

static constexpr size_t kLdsBudget = 160 * 1024;

size_t scan_lds_bytes(int mode_p, int nch, int k, int lut_queries) {
    const size_t lists = size_t(k) * kScanThreads * 8 + kQTile * sizeof(int) + (mode_p ? kDecodeBytes : 0);
    if (mode_p) {
        const size_t w = size_t(nch) * 2048;
        return (w + lists <= kLdsBudget ? w : 0) + lists;
    }
    return size_t(nch) * 1024 * lut_queries + lists;
}

// Workgroup size of the append-mode permute-dot scan (sample-then-filter, up to 32 queries).  The
// scan streams fastest with sixteen waves per CU on ONE copy of the query tile's weights in LDS:
// a 1024-thread workgroup of four four-wave groups, each group with a candidate segment of its own
// (the selection kernel reads short segments fastest).  Four-wave workgroups with a copy each (48 KiB
// at 1536 dimensions) reach twelve waves per CU where three copies fit -- one query over 10M x 1536
// bytes of codes at 128 to 1792 dimensions: 0.61-0.93 ms, the large workgroup 0.60-0.91, up to 18 %
// less -- and four waves per CU from 2560 dimensions (0.88 ms against 0.60).  Rows whose weights do
// not fit LDS (beyond 5056 dimensions) read them from global memory in four-wave workgroups.
constexpr int kScanThreadsShared = 4 * kScanThreads;
static int scan_p4_append_threads(int nch) {
    const size_t lds = size_t(nch) * 2048 + kDecodeBytes + (kScanThreadsShared / kScanThreads) * kQTile * sizeof(int);
    return lds <= kLdsBudget ? kScanThreadsShared : kScanThreads;
}

int scan_grid_blocks(int device, int mode_p, int nch, int k, int nq_tile) {
    hipDeviceProp_t prop;
    int cus = 256;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        cus = prop.multiProcessorCount;
    if (mode_p && k == 0 && scan_p4_append_threads(nch) != kScanThreads)           // (k = 0: the append-mode scans)
        return cus * (kScanThreadsShared / kScanThreads);                         // one workgroup per CU, counted in four-wave groups
    const size_t lds = scan_lds_bytes(mode_p, nch, k, nq_tile);
    int per_cu = int(kLdsBudget / (lds ? lds : 1));
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 4) per_cu = 4;
    // (the instances that read four or eight chunks per burst hold three waves per SIMD: a fourth
    // workgroup per CU would only wait for a place and run as a tail)
    if (mode_p && k == 0 && nch % 4 == 0 && per_cu > 3) per_cu = 3;
    return cus * per_cu;
}

hipError_t launch_scan_p4(const ScanArgs &args, int grid, int mode, hipStream_t s) {
    ScanArgs a = args;
    const int threads = (mode == kModeAppend || mode == kModeBest) ? scan_p4_append_threads(a.nch) : kScanThreads;
    const int groups = threads / kScanThreads;
    a.vgrid = uint32_t(grid);                        // `grid` counts four-wave groups
    const int wgs = (grid + groups - 1) / groups;
    const size_t w = size_t(a.nch) * 2048;
    const size_t lists = kDecodeBytes + groups * kQTile * sizeof(int) + (mode != kModeLists ? 0 : size_t(a.k) * kScanThreads * 8);
    const bool w_lds = w + lists <= kLdsBudget;
    const size_t lds = (w_lds ? w : 0) + lists;
    // (append-mode scans whose weights fit LDS take the large workgroup; four-wave ones read them from global memory)
    if ((mode == kModeAppend || mode == kModeBest) && groups == 1 && w_lds) return hipErrorInvalidValue;
    hipError_t e = hipSuccess;
#define TV_LAUNCH_P4_T(U, D, W, T)                                                              \
    do {                                                                                        \
        e = allow_lds(k_scan_p4<U, D, W, T>, lds);                                              \
        if (e != hipSuccess) return e;                                                          \
        hipLaunchKernelGGL((k_scan_p4<U, D, W, T>), dim3(wgs), dim3(T), lds, s, a);             \
    } while (0)
#define TV_LAUNCH_P4(U, D, W) TV_LAUNCH_P4_T(U, D, W, kScanThreads)
// (sixteen waves per CU leave a wave 128 registers: the large workgroup reads bursts of four chunks
// at most, and its floorless level -- a short launch either way -- of two)
#define TV_PICK_P4(U)                                                                           \
    do {                                                                                        \
        if (groups > 1) { if (mode == kModeAppend) TV_LAUNCH_P4_T((U > 4 ? 4 : U), kModeAppend, true, kScanThreadsShared); else TV_LAUNCH_P4_T((U > 2 ? 2 : U), kModeBest, true, kScanThreadsShared); } \
        else if (mode == kModeDump) { if (w_lds) TV_LAUNCH_P4(U, kModeDump, true); else TV_LAUNCH_P4(U, kModeDump, false); } \
        else if (mode == kModeAppend) TV_LAUNCH_P4(U, kModeAppend, false);                      \
        else if (mode == kModeBest) TV_LAUNCH_P4(U, kModeBest, false);                          \
        else { if (w_lds) TV_LAUNCH_P4(U, kModeLists, true); else TV_LAUNCH_P4(U, kModeLists, false); } \
    } while (0)
    if (a.nch % 8 == 0) TV_PICK_P4(8);          // 8 KiB per wave in flight: +3 % over 4 at 24 chunks, 12 is slower
    else if (a.nch % 4 == 0) TV_PICK_P4(4);
    else if (a.nch % 2 == 0) TV_PICK_P4(2);
    else TV_PICK_P4(1);
#undef TV_PICK_P4
#undef TV_LAUNCH_P4
#undef TV_LAUNCH_P4_T
    return hipGetLastError();
}

// Batched append-mode launches for up to batched_tiles()*32 queries (a.nq_tile counts queries,
// a.tables holds ceil(nq/32) consecutive tiles).  Two kernels: when the weights of at least two
// tiles fit LDS together they stay resident (k_scan_p4_multi); wider rows stream four tiles'
// weights through LDS in slices (k_scan_p4_batched).

// Query tiles whose weights fit LDS together, capped at 4.
// LDS of the resident-weights kernel beside nt tiles' weights: the byte table, the candidate
// counters and the block counter, 24 bytes of constants per query, a block's row scales per wave.
static size_t multi_fixed_lds(int nt) { return kDecodeBytes + (size_t(nt) * kQTile + 4) * sizeof(uint32_t) + size_t(nt) * kQTile * 24 + 16 * 32 * sizeof(float); }
static int resident_tiles(int nch) {
    const size_t per_tile = size_t(nch) * 2048;
    for (int nt = 4; nt >= 1; --nt)
        if (nt * per_tile + multi_fixed_lds(nt) <= kLdsBudget) return nt;
    return 0;
}

// Waves per workgroup of the resident-weights kernel and code bytes per lane and chunk it decodes
// through the table.  Four tiles: three waves per SIMD (measured best of 512 / 768 / 1024 threads),
// eight table bytes.  Two tiles fit 128 registers and run four waves per SIMD (2 to 7 % faster per
// launch, 256 to 2048 dimensions).  Three tiles fit them with four table bytes -- fewer reads in
// flight, fewer registers; by itself that split is 1 % slower -- and gain 1 to 3 % from the fourth wave.
template <int NT> constexpr int kMultiTableBytes = NT == 3 ? 4 : 8;
template <int NT> constexpr int kMultiThreads = NT <= 3 ? 1024 : 768;
constexpr int kStreamTiles = 4, kStreamBlocksPerWave = 2, kStreamSliceChunks = 2, kStreamOccupancy = 2;

// The resident-weights kernel reads its weights in k_scan_p4's split order.
bool batched_weights_split(int nch) { return resident_tiles(nch) >= 2; }

int batched_tiles(int nch) {
    const int nt = resident_tiles(nch);
    if (nt >= 2) return nt;
    return nch % kStreamSliceChunks == 0 ? kStreamTiles : 0;
}

int batched_grid_blocks(int device, int nch) {
    hipDeviceProp_t prop;
    int cus = 256;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        cus = prop.multiProcessorCount;
    if (resident_tiles(nch) >= 2) {
        const size_t lds = size_t(resident_tiles(nch)) * nch * 2048 + multi_fixed_lds(resident_tiles(nch));
        const int per_cu = int(kLdsBudget / lds);
        return cus * (per_cu < 1 ? 1 : (per_cu > 2 ? 2 : per_cu));
    }
    return cus * kStreamOccupancy;
}

template <int NT, int U>
static hipError_t launch_multi_u(const ScanArgs &a, int grid, hipStream_t s) {
    constexpr int LB = kMultiTableBytes<NT>;
    const size_t lds = size_t(NT) * a.nch * 2048 + multi_fixed_lds(NT);
    hipError_t e = allow_lds(k_scan_p4_multi<NT, U, kMultiThreads<NT>, LB>, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((k_scan_p4_multi<NT, U, kMultiThreads<NT>, LB>), dim3(grid), dim3(kMultiThreads<NT>), lds, s, a);
    return hipGetLastError();
}

template <int NT>
static hipError_t launch_multi(const ScanArgs &a, int grid, hipStream_t s) {
    // (four tiles' accumulators and four-chunk bursts together do not fit the 168 registers three
    // waves per SIMD leave: the compiler would spill, which the hand-placed waits cannot allow)
    if constexpr (NT < 4) {
        if (a.nch % 4 == 0) return launch_multi_u<NT, 4>(a, grid, s);
    }
    if (a.nch % 2 == 0) return launch_multi_u<NT, 2>(a, grid, s);
    return launch_multi_u<NT, 1>(a, grid, s);
}

hipError_t launch_scan_p4_batched(const ScanArgs &a, int grid, hipStream_t s) {
    // the instance for the tiles the launch really has: a third resident tile of padding queries
    // would cost its MFMAs all the same
    const int tiles = std::max(2, (a.nq_tile + kQTile - 1) / kQTile);
    switch (std::min(resident_tiles(a.nch), tiles)) {
        case 4: return launch_multi<4>(a, grid, s);
        case 3: return launch_multi<3>(a, grid, s);
        case 2: return launch_multi<2>(a, grid, s);
        default: break;
    }
    constexpr int MW = kStreamBlocksPerWave, KC = kStreamSliceChunks, OCC = kStreamOccupancy;
    if (a.nch % KC != 0 || a.nq_tile > kStreamTiles * kQTile) return hipErrorInvalidValue;
    auto launch = [&](auto ntc) -> hipError_t {
        constexpr int NT = decltype(ntc)::value;
        const size_t lds = size_t(2) * NT * KC * 2048 + NT * kQTile * sizeof(uint32_t);
        hipError_t e = allow_lds(k_scan_p4_batched<NT, MW, KC, OCC>, lds);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((k_scan_p4_batched<NT, MW, KC, OCC>), dim3(grid), dim3(kScanThreads), lds, s, a);
        return hipGetLastError();
    };
    static_assert(kStreamTiles == 4, "one instance per tile count up to the stream's four");
    switch (tiles) {        // as above: no tile of padding queries
        case 2: return launch(IntC<2>{});
        case 3: return launch(IntC<3>{});
        default: return launch(IntC<4>{});
    }
}

hipError_t launch_merge(const float *part_scores, const uint32_t *part_idx, const int *part_cnt, int total_threads,
                        int qmod, int k, int k_eff, int nq_tile, float *out_scores, int64_t *out_idx,
                        int *out_tau, hipStream_t s) {
    if (nq_tile == 0 || k_eff == 0) return hipSuccess;
    int sort_n = 2;
    while (sort_n < 256 * k) sort_n <<= 1;
    const size_t lds = size_t(k) * 256 * 8 + size_t(sort_n) * 8;
    hipError_t e = allow_lds(k_merge, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(k_merge, dim3(nq_tile), dim3(256), lds, s, part_scores, part_idx, part_cnt, total_threads,
                       qmod, k, k_eff, sort_n, out_scores, out_idx, out_tau);
    return hipGetLastError();
}

hipError_t launch_final(const uint64_t *cand, const uint32_t *cand_cnt, uint32_t n_seg, uint32_t seg_stride,
                        int k_eff, int k_floor, int nq, float *out_scores, int64_t *out_idx, uint32_t *overflow,
                        int *tau_out, int tau_stride_q, int keep_floor, int *raise_out, const uint32_t *row_map,
                        uint32_t *level_over, uint32_t *clear_flag, const uint32_t *run_if, hipStream_t s) {
    if (nq == 0 || k_eff == 0) return hipSuccess;
    hipLaunchKernelGGL(k_final, dim3(nq), dim3(kFinalThreads), 0, s, cand, cand_cnt, n_seg, seg_stride, k_eff, k_floor,
                       out_scores, out_idx, overflow, tau_out, tau_stride_q, keep_floor, raise_out, row_map, level_over,
                       clear_flag, run_if);
    return hipGetLastError();
}

}  // namespace tv
