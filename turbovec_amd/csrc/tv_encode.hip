// Ingest: encode raw float rows on the device and append them to the index.
//
// One workgroup per row.  Every float operation is the one the reference does,
// in the reference's order, so codes and scales are bit-identical to the CPU
// encoder's (turbovec/src/encode.rs:1418-1476 encode_batch_chunk, :560-664
// quantize, :900-932 norm; turbovec/src/rotation.rs:218-255 apply_scaled_into):
//   * the squared norm runs in 8 interleaved f32 chains (element j feeds chain
//     j % 8), folded pairwise; each chain is sequential, so 8 lanes carry them;
//   * the rotation is the query rotation with the 1/norm folded into the first
//     gather: (x[perm0[i]] * inv) * sign0[i];
//   * the reconstruction inner product runs in 4 interleaved f64 chains
//     (element j feeds chain j % 4), folded pairwise; 4 lanes carry them.
// Only the additions of those chains are sequential: the squares and the f64
// products they add up are computed by all threads first, each by the same
// operations as in the reference, and parked in LDS.
#include <hip/hip_runtime.h>

#include "tv_internal.h"

namespace tv {

struct EncodeArgs {
    const float *vecs;        // n_new * dim raw rows (device)
    const float *signs;       // 2 * dim
    const uint32_t *perms;    // 2 * dim
    const float *shift;       // dim, or nullptr for the identity pair (encode.rs:578-590)
    const float *scale;       // dim, or nullptr
    float cen[16];
    float bnd[16];
    int dim, bits, G, nch, block;
    float inv_sqrt_block;
    float *rot_out;           // when set: write the rotated unit rows here and stop (TQ+ fit input)
    uint8_t *nat;             // codes in the device layout
    float *scales;
    size_t old_n, n_new;
};

__device__ __forceinline__ size_t enc_byte_index(size_t v, int g, int nch) {
    const size_t b = v >> 5;
    const int i = int(v & 31);
    return ((b * size_t(nch) + size_t(g >> 5)) * 64 + size_t(((g & 31) >> 4) * 32 + i)) * 16 + size_t(g & 15);
}

__device__ __forceinline__ void wht_lds(float *x, int dim, int block, int t) {
    for (int len = 1; len < block; len <<= 1) {
        for (int p = t; p < dim / 2; p += 256) {
            const int j = 2 * p - (p & (len - 1));
            const float a = x[j], b = x[j + len];
            x[j] = a + b;
            x[j + len] = a - b;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void k_encode(EncodeArgs a) {
    extern __shared__ __align__(16) float enc_lds[];
    const int dim = a.dim, t = threadIdx.x;
    float *A = enc_lds;
    float *B = enc_lds + dim;
    __shared__ float red[8];
    __shared__ double dred[4];
    __shared__ float s_cen[16];
    const size_t row = blockIdx.x;
    const float *src = a.vecs + row * size_t(dim);
    if (t < 16) s_cen[t] = a.cen[t];
    for (int i = t; i < dim; i += 256) A[i] = src[i];
    __syncthreads();

    // encode.rs:920-932: c[j % 8] += x * x (separate multiply and add), then the pairwise fold
    for (int i = t; i < dim; i += 256) B[i] = A[i] * A[i];
    __syncthreads();
    if (t < 8) {
        float c = 0.0f;
        for (int j = t; j < dim; j += 8) c = c + B[j];
        red[t] = c;
    }
    __syncthreads();
    const float nrm = sqrtf(((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7])));
    const float inv = nrm > 1e-10f ? 1.0f / nrm : 0.0f;   // lib.rs:163 MIN_INPUT_NORM

    for (int i = t; i < dim; i += 256) B[i] = (A[a.perms[i]] * inv) * a.signs[i];
    __syncthreads();
    wht_lds(B, dim, a.block, t);
    for (int i = t; i < dim; i += 256) A[i] = (B[a.perms[dim + i]] * a.inv_sqrt_block) * a.signs[dim + i];
    __syncthreads();
    wht_lds(A, dim, a.block, t);
    for (int i = t; i < dim; i += 256) B[i] = A[i] * a.inv_sqrt_block;   // B = rotated unit row
    __syncthreads();
    if (a.rot_out != nullptr) {
        float *dst = a.rot_out + row * size_t(dim);
        for (int i = t; i < dim; i += 256) dst[i] = B[i];
        return;
    }

    // encode.rs:600-640: code = number of boundaries below the calibrated value
    uint8_t *codes = reinterpret_cast<uint8_t *>(A);
    const int nb = (1 << a.bits) - 1;
    for (int i = t; i < dim; i += 256) {
        const float sh = a.shift ? a.shift[i] : 0.0f;
        const float sc = a.scale ? a.scale[i] : 1.0f;
        const float calib = (B[i] + sh) * sc;
        int v = 0;
        for (int b = 0; b < nb; ++b) v += calib > a.bnd[b] ? 1 : 0;
        codes[i] = uint8_t(v);
    }
    __syncthreads();

    // encode.rs:1442-1475: inner = <rotated, reconstruction> in f64, four chains by j % 4.
    // The f64 products are parked piece by piece in what is left of A behind the codes
    // (3 * dim bytes), so the kernel needs 8 * dim bytes of LDS whatever the row length; a
    // chain walks its elements in rising order across the pieces, as in one sweep.
    // (rows of 8 dimensions leave no room for one product per chain there: they use the four
    // spare doubles behind B)
    const int piece = dim >= 16 ? (3 * dim / 8) & ~3 : 4;
    double *terms = dim >= 16 ? reinterpret_cast<double *>(reinterpret_cast<uint8_t *>(A) + dim)
                              : reinterpret_cast<double *>(enc_lds + 2 * dim);
    double ch = 0.0;
    for (int j0 = 0; j0 < dim; j0 += piece) {
        const int j1 = min(dim, j0 + piece);
        for (int j = j0 + t; j < j1; j += 256) {
            const float sh = a.shift ? a.shift[j] : 0.0f;
            const float sc = a.scale ? a.scale[j] : 1.0f;
            const float inv_sc = 1.0f / sc;                       // encode.rs:594
            const double recon = double(s_cen[codes[j]]) * double(inv_sc) - double(sh);
            terms[j - j0] = double(B[j]) * recon;
        }
        __syncthreads();
        if (t < 4)
            for (int j = j0 + t; j < j1; j += 4) ch = ch + terms[j - j0];
        __syncthreads();
    }
    if (t < 4) dred[t] = ch;
    __syncthreads();
    if (t == 0) {
        const double inner = (dred[0] + dred[1]) + (dred[2] + dred[3]);
        a.scales[a.old_n + row] = inner > 0.1 ? nrm / float(inner) : 0.0f;   // encode.rs:1194-1200
    }

    // pack.rs:264-282 byte of a group (first dimension in the high bits; 3-bit codes sit in
    // 4-bit fields), written at the row's lane of the device layout (pack.rs:211-233 append_lanes)
    const int cpb = a.bits == 2 ? 4 : 2;
    const int field = a.bits == 2 ? 2 : 4;
    for (int g = t; g < a.G; g += 256) {
        unsigned byte = 0;
        for (int c = 0; c < cpb; ++c) byte |= unsigned(codes[g * cpb + c]) << ((cpb - 1 - c) * field);
        a.nat[enc_byte_index(a.old_n + row, g, a.nch)] = uint8_t(byte);
    }
}

// A and B, one float row each; codes and the f64 products overlay A.  128 KiB at the largest
// row the index accepts (16384 dimensions), inside the 160 KiB a workgroup may have.
static_assert(size_t(2) * 16384 * sizeof(float) + 4 * sizeof(double) <= 160 * 1024,
              "the longest row the index accepts (lib.rs:101 MAX_DIM) must fit a workgroup's LDS");
size_t encode_lds_bytes(int dim) { return size_t(2) * size_t(dim) * sizeof(float) + 4 * sizeof(double); }

hipError_t launch_encode(const float *d_vecs, size_t n_new, size_t old_n, const float *d_signs,
                         const uint32_t *d_perms, const float *d_shift, const float *d_scale,
                         const float *centroids, const float *boundaries, const Geometry &g, int block,
                         float inv_sqrt_block, uint8_t *d_native, float *d_scales, float *d_rot_out,
                         hipStream_t s) {
    if (n_new == 0) return hipSuccess;
    EncodeArgs a;
    a.vecs = d_vecs; a.signs = d_signs; a.perms = d_perms; a.shift = d_shift; a.scale = d_scale;
    const int nl = 1 << g.bits;
    for (int i = 0; i < 16; ++i) { a.cen[i] = i < nl ? centroids[i] : 0.0f; a.bnd[i] = i < nl - 1 ? boundaries[i] : 0.0f; }
    a.dim = g.dim; a.bits = g.bits; a.G = g.G; a.nch = g.nch; a.block = block;
    a.inv_sqrt_block = inv_sqrt_block;
    a.nat = d_native; a.scales = d_scales; a.old_n = old_n; a.n_new = n_new;
    a.rot_out = d_rot_out;
    const size_t lds = encode_lds_bytes(g.dim);
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_encode),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(k_encode, dim3(unsigned(n_new)), dim3(256), lds, s, a);
    return hipGetLastError();
}

}  // namespace tv
