/*
 * tv_oracle.c -- CPU restatement of the turbovec search path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP search path.  See
 * tv_oracle.h for the parity status of every function.  Build with
 * -ffp-contract=off: every float expression below relies on separate IEEE
 * multiplies and adds exactly where the reference has them, and on fmaf only
 * where the reference fuses.
 */
#include "tv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ======================================================================= */
/* ChaCha8 -- rand_chacha =0.3.1 ChaCha8Rng (turbovec/Cargo.toml:49).       */
/* The dependency's source is not in the reference tree; this is the        */
/* published ChaCha block function with 8 rounds, a 64-bit block counter in */
/* words 12-13, a zero stream id in words 14-15, and rand_core's BlockRng   */
/* buffering of four blocks (64 words) per refill.  Arbiter: the rotation   */
/* goldens (turbovec/tests/rotation_determinism.rs:75-96).                  */
/* ======================================================================= */

static inline uint32_t rotl32(uint32_t x, int n) { return (x << n) | (x >> (32 - n)); }

#define QR(a, b, c, d)            \
    do {                          \
        a += b; d ^= a; d = rotl32(d, 16); \
        c += d; b ^= c; b = rotl32(b, 12); \
        a += b; d ^= a; d = rotl32(d, 8);  \
        c += d; b ^= c; b = rotl32(b, 7);  \
    } while (0)

static void chacha8_block(const uint32_t key[8], uint64_t counter, uint32_t out[16]) {
    uint32_t in[16], x[16];
    in[0] = 0x61707865u; in[1] = 0x3320646eu; in[2] = 0x79622d32u; in[3] = 0x6b206574u;
    for (int i = 0; i < 8; i++) in[4 + i] = key[i];
    in[12] = (uint32_t)counter;
    in[13] = (uint32_t)(counter >> 32);
    in[14] = 0;
    in[15] = 0;
    memcpy(x, in, sizeof x);
    for (int dr = 0; dr < 4; dr++) { /* 8 rounds = 4 double rounds */
        QR(x[0], x[4], x[8], x[12]);
        QR(x[1], x[5], x[9], x[13]);
        QR(x[2], x[6], x[10], x[14]);
        QR(x[3], x[7], x[11], x[15]);
        QR(x[0], x[5], x[10], x[15]);
        QR(x[1], x[6], x[11], x[12]);
        QR(x[2], x[7], x[8], x[13]);
        QR(x[3], x[4], x[9], x[14]);
    }
    for (int i = 0; i < 16; i++) out[i] = x[i] + in[i];
}

void tvo_chacha8_init(tvo_chacha8 *rng, const uint8_t seed[32]) {
    for (int i = 0; i < 8; i++) {
        rng->key[i] = (uint32_t)seed[4 * i] | ((uint32_t)seed[4 * i + 1] << 8) |
                      ((uint32_t)seed[4 * i + 2] << 16) | ((uint32_t)seed[4 * i + 3] << 24);
    }
    rng->counter = 0;
    rng->index = 64;
}

static void chacha8_refill(tvo_chacha8 *rng) {
    for (int b = 0; b < 4; b++) chacha8_block(rng->key, rng->counter + (uint64_t)b, rng->buf + 16 * b);
    rng->counter += 4;
    rng->index = 0;
}

uint32_t tvo_chacha8_next_u32(tvo_chacha8 *rng) {
    if (rng->index >= 64) chacha8_refill(rng);
    return rng->buf[rng->index++];
}

/* rand_core 0.6 BlockRng::next_u64: low word first; the one-word-left case
 * takes the last word as the low half, refills, and takes word 0 as the high. */
uint64_t tvo_chacha8_next_u64(tvo_chacha8 *rng) {
    if (rng->index < 63) {
        uint64_t lo = rng->buf[rng->index], hi = rng->buf[rng->index + 1];
        rng->index += 2;
        return (hi << 32) | lo;
    } else if (rng->index == 63) {
        uint64_t lo = rng->buf[63];
        chacha8_refill(rng);
        uint64_t hi = rng->buf[0];
        rng->index = 1;
        return (hi << 32) | lo;
    } else {
        chacha8_refill(rng);
        uint64_t lo = rng->buf[0], hi = rng->buf[1];
        rng->index = 2;
        return (hi << 32) | lo;
    }
}

/* ======================================================================= */
/* Rotation -- turbovec/src/rotation.rs                                     */
/* ======================================================================= */

/* rotation.rs:82-85 ROTATION_SEED */
static const uint8_t ROTATION_SEED[32] = {
    164, 143, 161, 123, 88, 50, 61, 10, 234, 184, 161, 204, 105, 1, 20, 184,
    43, 140, 200, 117, 24, 180, 247, 84, 141, 68, 110, 161, 228, 223, 32, 242};

/* rotation.rs:141-187 Rotation::new; fisher_yates rotation.rs:990-997 */
tvo_rotation *tvo_rotation_new(int dim) {
    if (dim <= 0 || dim % 8 != 0 || dim > TVO_MAX_DIM) return NULL;
    tvo_rotation *r = (tvo_rotation *)calloc(1, sizeof *r);
    r->dim = dim;
    r->block = dim & (-dim); /* rotation.rs:92-95 largest power-of-two divisor */
    r->inv_sqrt_block = 1.0f / sqrtf((float)r->block);
    tvo_chacha8 rng;
    tvo_chacha8_init(&rng, ROTATION_SEED);
    for (int round = 0; round < 2; round++) {
        r->signs[round] = (float *)malloc(sizeof(float) * (size_t)dim);
        r->perms[round] = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)dim);
        for (int i = 0; i < dim; i++)
            r->signs[round][i] = (tvo_chacha8_next_u32(&rng) & 1u) ? -1.0f : 1.0f;
        uint32_t *p = r->perms[round];
        for (int i = 0; i < dim; i++) p[i] = (uint32_t)i;
        for (int i = dim - 1; i >= 1; i--) {
            uint64_t j = tvo_chacha8_next_u64(&rng) % ((uint64_t)i + 1);
            uint32_t t = p[i]; p[i] = p[j]; p[j] = t;
        }
    }
    return r;
}

void tvo_rotation_free(tvo_rotation *r) {
    if (!r) return;
    for (int i = 0; i < 2; i++) { free(r->signs[i]); free(r->perms[i]); }
    free(r);
}

int tvo_rotation_block(const tvo_rotation *r) { return r->block; }
const float *tvo_rotation_signs(const tvo_rotation *r, int round) { return r->signs[round]; }
const uint32_t *tvo_rotation_perm(const tvo_rotation *r, int round) { return r->perms[round]; }

/* rotation.rs:964-982 wht_block_scalar */
static void wht_block(float *blk, int block, float inv_sqrt_block) {
    for (int len = 1; len < block; len <<= 1) {
        for (int i = 0; i < block; i += 2 * len) {
            for (int j = i; j < i + len; j++) {
                float a = blk[j], b = blk[j + len];
                blk[j] = a + b;
                blk[j + len] = a - b;
            }
        }
    }
    for (int i = 0; i < block; i++) blk[i] *= inv_sqrt_block;
}

/* rotation.rs:265-320 apply_with_scratch (ping-pong, K = 2) */
void tvo_rotation_apply(const tvo_rotation *r, float *row) {
    int dim = r->dim;
    float *scratch = (float *)malloc(sizeof(float) * (size_t)dim);
    float *in = row, *out = scratch;
    for (int round = 0; round < 2; round++) {
        const uint32_t *perm = r->perms[round];
        const float *sg = r->signs[round];
        for (int i = 0; i < dim; i++) out[i] = in[perm[i]] * sg[i];
        for (int off = 0; off < dim; off += r->block) wht_block(out + off, r->block, r->inv_sqrt_block);
        float *t = in; in = out; out = t;
    }
    free(scratch);
}

/* rotation.rs:218-255 apply_scaled_into: round 0 gathers (src*inv)*sign. */
void tvo_rotation_apply_scaled(const tvo_rotation *r, const float *src, float inv, float *dst) {
    int dim = r->dim;
    float *scratch = (float *)malloc(sizeof(float) * (size_t)dim);
    for (int i = 0; i < dim; i++) scratch[i] = (src[r->perms[0][i]] * inv) * r->signs[0][i];
    for (int off = 0; off < dim; off += r->block) wht_block(scratch + off, r->block, r->inv_sqrt_block);
    for (int i = 0; i < dim; i++) dst[i] = scratch[r->perms[1][i]] * r->signs[1][i];
    for (int off = 0; off < dim; off += r->block) wht_block(dst + off, r->block, r->inv_sqrt_block);
    free(scratch);
}

/* ======================================================================= */
/* Beta(a,a) cdf/pdf -- statrs =0.17.1 (turbovec/Cargo.toml:67), source not  */
/* in the reference tree.  Published algorithm: regularized incomplete beta  */
/* by the modified-Lentz continued fraction with the symmetry swap.          */
/* Arbiter: the codebook FNV goldens.                                        */
/* ======================================================================= */

static double beta_reg(double a, double b, double x) {
    double bt;
    if (x == 0.0 || x == 1.0) bt = 0.0;
    else bt = exp(lgamma(a + b) - lgamma(a) - lgamma(b) + a * log(x) + b * log(1.0 - x));
    int symm = x >= (a + 1.0) / (a + b + 2.0);
    const double eps = 1.1102230246251565e-16;
    const double fpmin = DBL_MIN / eps;
    if (symm) { double t = a; a = b; b = t; x = 1.0 - x; }
    double qab = a + b, qap = a + 1.0, qam = a - 1.0;
    double c = 1.0, d = 1.0 - qab * x / qap;
    if (fabs(d) < fpmin) d = fpmin;
    d = 1.0 / d;
    double h = d;
    for (int mi = 1; mi < 141; mi++) {
        double m = (double)mi, m2 = m * 2.0;
        double aa = m * (b - m) * x / ((qam + m2) * (a + m2));
        d = 1.0 + aa * d;
        if (fabs(d) < fpmin) d = fpmin;
        c = 1.0 + aa / c;
        if (fabs(c) < fpmin) c = fpmin;
        d = 1.0 / d;
        h = h * d * c;
        aa = -(a + m) * (qab + m) * x / ((a + m2) * (qap + m2));
        d = 1.0 + aa * d;
        if (fabs(d) < fpmin) d = fpmin;
        c = 1.0 + aa / c;
        if (fabs(c) < fpmin) c = fpmin;
        d = 1.0 / d;
        double del = d * c;
        h *= del;
        if (fabs(del - 1.0) <= eps) break;
    }
    return symm ? 1.0 - bt * h / a : bt * h / a;
}

double tvo_beta_cdf(double a, double x) {
    if (x < 0.0) return 0.0;
    if (x >= 1.0) return 1.0;
    return beta_reg(a, a, x);
}

double tvo_beta_pdf(double a, double x) {
    if (!(x >= 0.0 && x <= 1.0)) return 0.0;
    if (a > 80.0) {
        double aa = lgamma(a + a) - lgamma(a) - lgamma(a);
        double bb = (x == 0.0) ? -INFINITY : (a - 1.0) * log(x);
        double cc = (x == 1.0) ? -INFINITY : (a - 1.0) * log(1.0 - x);
        return exp(aa + bb + cc);
    }
    double bb = tgamma(a + a) / (tgamma(a) * tgamma(a));
    return bb * pow(x, a - 1.0) * pow(1.0 - x, a - 1.0);
}

/* ======================================================================= */
/* Codebook -- turbovec/src/codebook.rs:69-167, adaptive Simpson 214-249    */
/* ======================================================================= */

typedef struct { double a; } pdf_ctx;

static double shifted_mean_integrand(const pdf_ctx *c, double x) {
    double t = (x + 1.0) / 2.0;
    return x * tvo_beta_pdf(c->a, t) / 2.0;
}

static double simpson_rec(const pdf_ctx *c, double a, double b, double fa, double fb, double fm,
                          double whole, double tol, int depth) {
    double mid = (a + b) / 2.0;
    double m1 = (a + mid) / 2.0, m2 = (mid + b) / 2.0;
    double fm1 = shifted_mean_integrand(c, m1), fm2 = shifted_mean_integrand(c, m2);
    double left = (mid - a) / 6.0 * (fa + 4.0 * fm1 + fm);
    double right = (b - mid) / 6.0 * (fm + 4.0 * fm2 + fb);
    double refined = left + right;
    if (depth == 0 || fabs(refined - whole) < 15.0 * tol) return refined + (refined - whole) / 15.0;
    return simpson_rec(c, a, mid, fa, fm, fm1, left, tol / 2.0, depth - 1) +
           simpson_rec(c, mid, b, fm, fb, fm2, right, tol / 2.0, depth - 1);
}

static double adaptive_simpson(const pdf_ctx *c, double a, double b, double tol, int max_depth) {
    double mid = (a + b) / 2.0;
    double fa = shifted_mean_integrand(c, a), fb = shifted_mean_integrand(c, b);
    double fm = shifted_mean_integrand(c, mid);
    double whole = (b - a) / 6.0 * (fa + 4.0 * fm + fb);
    return simpson_rec(c, a, b, fa, fb, fm, whole, tol, max_depth);
}

int tvo_codebook(int bits, int dim, float *boundaries, float *centroids) {
    if (bits < 2 || bits > 4 || dim < 2) return TVO_ERR_BAD_ARGUMENT;
    double a = ((double)dim - 1.0) / 2.0;
    pdf_ctx ctx = {a};
    int L = 1 << bits;
    double cen[16], nc[16], edges[17];
    double std_dev = sqrt(2.0 * a / ((2.0 * a + 1.0) * 4.0 * a));
    double spread = 3.0 * std_dev;
    for (int i = 0; i < L; i++) cen[i] = -spread + 2.0 * spread * (double)i / ((double)L - 1.0);
    for (int iter = 0; iter < 200; iter++) {
        edges[0] = -1.0;
        for (int i = 0; i < L - 1; i++) edges[i + 1] = (cen[i] + cen[i + 1]) / 2.0;
        edges[L] = 1.0;
        for (int i = 0; i < L; i++) {
            double lo = edges[i], hi = edges[i + 1];
            double prob = tvo_beta_cdf(a, (hi + 1.0) / 2.0) - tvo_beta_cdf(a, (lo + 1.0) / 2.0);
            if (prob < 1e-15) nc[i] = cen[i];
            else nc[i] = adaptive_simpson(&ctx, lo, hi, 1e-14, 50) / prob;
        }
        double max_change = 0.0;
        for (int i = 0; i < L; i++) {
            double ch = fabs(cen[i] - nc[i]);
            if (ch > max_change) max_change = ch;
            cen[i] = nc[i];
        }
        if (max_change < 1e-12) break;
    }
    for (int i = 0; i < L; i++) centroids[i] = (float)cen[i];
    for (int i = 0; i < L - 1; i++) boundaries[i] = (centroids[i] + centroids[i + 1]) * 0.5f;
    return TVO_OK;
}

/* ======================================================================= */
/* Encode -- turbovec/src/encode.rs                                         */
/* ======================================================================= */

/* encode.rs:920-932 norm_sq_scalar + combine tree, then sqrt (900-918) */
float tvo_norm(const float *row, int dim) {
    float c[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = 0; j < dim; j++) c[j % 8] += row[j] * row[j];
    float s = ((c[0] + c[1]) + (c[2] + c[3])) + ((c[4] + c[5]) + (c[6] + c[7]));
    return sqrtf(s);
}

/* encode.rs:183-186 f32_sort_key */
static inline uint32_t f32_sort_key(float x) {
    uint32_t b; memcpy(&b, &x, 4);
    return b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
}
static inline float f32_from_sort_key(uint32_t k) {
    uint32_t m = (k & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu;
    uint32_t b = k ^ m; float x; memcpy(&x, &b, 4); return x;
}
static int cmp_u32(const void *a, const void *b) {
    uint32_t x = *(const uint32_t *)a, y = *(const uint32_t *)b;
    return (x > y) - (x < y);
}

/* rotate_batch_into encode.rs:406-458 for one row: norm, inv, rotate scaled */
static float rotate_row_normalised(const tvo_rotation *r, const float *src, float *dst) {
    float nrm = tvo_norm(src, r->dim);
    float inv = nrm > 1e-10f ? 1.0f / nrm : 0.0f; /* lib.rs:163 MIN_INPUT_NORM */
    tvo_rotation_apply_scaled(r, src, inv, dst);
    return nrm;
}

/* encode.rs:737-857 compute_tqplus_calibration (+ tqplus_anchor 364-369) */
void tvo_fit_calibration(const tvo_rotation *r, const float *vectors, size_t n, int dim,
                         const float *centroids, int n_levels, float *shift, float *scale) {
    float *rot = (float *)malloc(sizeof(float) * n * (size_t)dim);
    for (size_t i = 0; i < n; i++) rotate_row_normalised(r, vectors + i * dim, rot + i * dim);
    double a = ((double)dim - 1.0) / 2.0;
    float c_outer = 0.0f;
    for (int i = 0; i < n_levels; i++) { float v = fabsf(centroids[i]); if (v > c_outer) c_outer = v; }
    double p_hi = tvo_beta_cdf(a, ((double)c_outer + 1.0) / 2.0);
    double p_lo = 1.0 - p_hi;
    float qc_lo = -c_outer, qc_hi = c_outer;
    float qc_span = qc_hi - qc_lo;
    size_t lo_idx = (size_t)((double)n * p_lo);
    size_t hi_idx = (size_t)((double)n * p_hi);
    if (hi_idx > n - 1) hi_idx = n - 1;
    if (hi_idx < lo_idx + 1) hi_idx = lo_idx + 1;
    uint32_t *col = (uint32_t *)malloc(sizeof(uint32_t) * n);
    for (int d = 0; d < dim; d++) {
        shift[d] = 0.0f; scale[d] = 1.0f;
        for (size_t i = 0; i < n; i++) col[i] = f32_sort_key(rot[i * dim + d]);
        qsort(col, n, sizeof(uint32_t), cmp_u32);
        float qe_lo = f32_from_sort_key(col[lo_idx]);
        float qe_hi = f32_from_sort_key(col[hi_idx]);
        float qe_span = qe_hi - qe_lo;
        if (qe_span > 1e-6f) {
            scale[d] = qc_span / qe_span;
            shift[d] = qc_lo / scale[d] - qe_lo;
        }
    }
    free(col); free(rot);
}

/* encode.rs:1418-1476 fused_quantize_scale_pack_scalar; 1194-1200 scale_from_inner */
static float quantize_row(const float *rot, const float *shift, const float *scale_tq,
                          const float *inv_scale_tq, const float *boundaries, const float *centroids,
                          float norm, int bits, int dim, uint8_t *packed_row) {
    int bytes_per_plane = dim / 8;
    int nb = (1 << bits) - 1;
    double chains[4] = {0, 0, 0, 0};
    for (int c = 0; c < dim / 8; c++) {
        uint8_t codes[8];
        for (int k = 0; k < 8; k++) {
            int j = c * 8 + k;
            float calib = (rot[j] + shift[j]) * scale_tq[j];
            uint8_t v = 0;
            for (int bi = 0; bi < nb; bi++) if (calib > boundaries[bi]) v++;
            codes[k] = v;
            double recon = (double)centroids[v] * (double)inv_scale_tq[j] - (double)shift[j];
            chains[j % 4] += (double)rot[j] * recon;
        }
        for (int p = 0; p < bits; p++) {
            uint8_t byte = 0;
            for (int k = 0; k < 8; k++) byte |= (uint8_t)(((codes[k] >> p) & 1) << (7 - k));
            packed_row[p * bytes_per_plane + c] = byte;
        }
    }
    double inner = (chains[0] + chains[1]) + (chains[2] + chains[3]);
    return inner > 0.1 ? norm / (float)inner : 0.0f;
}

void tvo_encode(const tvo_rotation *r, const float *vectors, size_t n, int dim, int bits,
                const float *boundaries, const float *centroids,
                const float *shift_in, const float *scale_in,
                uint8_t *packed_out, float *scales_out) {
    float *shift = (float *)malloc(sizeof(float) * (size_t)dim);
    float *scale_tq = (float *)malloc(sizeof(float) * (size_t)dim);
    float *inv_scale = (float *)malloc(sizeof(float) * (size_t)dim);
    for (int d = 0; d < dim; d++) {
        shift[d] = shift_in ? shift_in[d] : 0.0f;    /* encode.rs:578-590 identity pair */
        scale_tq[d] = scale_in ? scale_in[d] : 1.0f;
        inv_scale[d] = 1.0f / scale_tq[d];           /* encode.rs:594 */
    }
    size_t bytes_per_row = (size_t)bits * (size_t)(dim / 8);
#pragma omp parallel
    {
        float *rot = (float *)malloc(sizeof(float) * (size_t)dim);
#pragma omp for schedule(static)
        for (long long i = 0; i < (long long)n; i++) {
            float nrm = rotate_row_normalised(r, vectors + (size_t)i * dim, rot);
            scales_out[i] = quantize_row(rot, shift, scale_tq, inv_scale, boundaries, centroids, nrm,
                                         bits, dim, packed_out + (size_t)i * bytes_per_row);
        }
        free(rot);
    }
    free(shift); free(scale_tq); free(inv_scale);
}

/* ======================================================================= */
/* Layouts -- turbovec/src/pack.rs                                          */
/* ======================================================================= */

size_t tvo_n_byte_groups(int bits, int dim) { return (size_t)dim / (size_t)(8 / bits); }

size_t tvo_seq_len(size_t n, int bits, int dim) {
    size_t n_blocks = (n + TVO_BLOCK - 1) / TVO_BLOCK;
    return n_blocks * tvo_n_byte_groups(bits, dim) * TVO_BLOCK;
}

/* Code of dimension j of one bit-plane packed row (encode.rs:1464-1470). */
static inline unsigned packed_code(const uint8_t *row, int bits, int bytes_per_plane, int j) {
    unsigned v = 0;
    for (int p = 0; p < bits; p++) v |= (unsigned)((row[p * bytes_per_plane + j / 8] >> (7 - (j % 8))) & 1) << p;
    return v;
}

/* pack.rs:264-282 (bit placement) + 336-361 (sequential blocked) = repack_seq :366 */
void tvo_repack_seq(const uint8_t *packed, size_t n, int bits, int dim, uint8_t *seq_out) {
    int cpb = 8 / bits;
    int field = bits == 3 ? 4 : bits;
    size_t G = tvo_n_byte_groups(bits, dim);
    int bytes_per_plane = dim / 8;
    size_t bytes_per_row = (size_t)bits * bytes_per_plane;
    memset(seq_out, 0, tvo_seq_len(n, bits, dim));
    for (size_t vi = 0; vi < n; vi++) {
        const uint8_t *row = packed + vi * bytes_per_row;
        size_t b = vi / TVO_BLOCK, lane = vi % TVO_BLOCK;
        for (size_t g = 0; g < G; g++) {
            unsigned byte = 0;
            for (int c = 0; c < cpb; c++) {
                unsigned code = packed_code(row, bits, bytes_per_plane, (int)(g * cpb + c));
                byte |= code << ((cpb - 1 - c) * field);
            }
            seq_out[(b * G + g) * TVO_BLOCK + lane] = (uint8_t)byte;
        }
    }
}

/* pack.rs:375-420 seq_to_packed */
void tvo_seq_to_packed(const uint8_t *seq, size_t n, int bits, int dim, uint8_t *packed_out) {
    int cpb = 8 / bits;
    int field = bits == 3 ? 4 : bits;
    size_t G = tvo_n_byte_groups(bits, dim);
    int bytes_per_plane = dim / 8;
    size_t bytes_per_row = (size_t)bits * bytes_per_plane;
    memset(packed_out, 0, n * bytes_per_row);
    for (size_t vi = 0; vi < n; vi++) {
        uint8_t *row = packed_out + vi * bytes_per_row;
        size_t b = vi / TVO_BLOCK, lane = vi % TVO_BLOCK;
        for (size_t g = 0; g < G; g++) {
            unsigned byte = seq[(b * G + g) * TVO_BLOCK + lane];
            for (int c = 0; c < cpb; c++) {
                unsigned code = (byte >> ((cpb - 1 - c) * field)) & ((1u << bits) - 1);
                int j = (int)(g * cpb + c);
                for (int p = 0; p < bits; p++)
                    if ((code >> p) & 1) row[p * bytes_per_plane + j / 8] |= (uint8_t)(1u << (7 - (j % 8)));
            }
        }
    }
}

/* lib.rs:2964-3003 + pack.rs:174-243 on the sequential layout */
size_t tvo_swap_remove_seq(uint8_t *seq, float *scales, size_t n, int bits, int dim, size_t idx) {
    size_t G = tvo_n_byte_groups(bits, dim);
    size_t last = n - 1;
    size_t sb = last / TVO_BLOCK, sl = last % TVO_BLOCK;
    if (idx != last) {
        size_t db = idx / TVO_BLOCK, dl = idx % TVO_BLOCK;
        for (size_t g = 0; g < G; g++) seq[(db * G + g) * TVO_BLOCK + dl] = seq[(sb * G + g) * TVO_BLOCK + sl];
        scales[idx] = scales[last];
    }
    for (size_t g = 0; g < G; g++) seq[(sb * G + g) * TVO_BLOCK + sl] = 0;
    return last;
}

/* ======================================================================= */
/* Query preparation -- turbovec/src/search.rs                              */
/* ======================================================================= */

/* Rust f32::round is round-half-away-from-zero == roundf. */
static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* search.rs:2856-2994 build_query_neon_lut_from_slice.  Sub-table at [g*32+0..16]
 * covers the group's first dims and is indexed by the byte's HIGH nibble
 * (search.rs:3124-3127); [g*32+16..32] covers the remaining dims (LOW nibble). */
void tvo_build_lut(const float *q, const float *centroids, int bits, int dim,
                   uint8_t *lut, float *scale_out, float *bias_out) {
    int cpb = 8 / bits;
    int cpn = cpb / 2;
    size_t G = (size_t)dim / (size_t)cpb;
    unsigned code_mask = (1u << bits) - 1;
    float *fv = (float *)malloc(sizeof(float) * G * 32);
    float *mins = (float *)malloc(sizeof(float) * G * 2);
    float max_span = 0.0f, bias = 0.0f;
    for (size_t g = 0; g < G; g++) {
        size_t dim_start = g * (size_t)cpb;
        float mn[2], mx[2];
        for (int sub = 0; sub < 2; sub++) {
            mn[sub] = FLT_MAX; mx[sub] = -FLT_MAX; /* f32::MAX / f32::MIN */
            for (unsigned nv = 0; nv < 16; nv++) {
                float s = 0.0f;
                for (int c = 0; c < cpn; c++) {
                    int sh = (cpn - 1 - c) * bits;
                    unsigned code = (nv >> sh) & code_mask;
                    s += q[dim_start + (size_t)(sub * cpn + c)] * centroids[code];
                }
                fv[g * 32 + (size_t)sub * 16 + nv] = s;
                if (s < mn[sub]) mn[sub] = s;
                if (s > mx[sub]) mx[sub] = s;
            }
        }
        mins[g * 2] = mn[0]; mins[g * 2 + 1] = mn[1];
        bias += mn[0] + mn[1];
        float s0 = mx[0] - mn[0], s1 = mx[1] - mn[1];
        if (s0 > max_span) max_span = s0;
        if (s1 > max_span) max_span = s1;
    }
    const float max_lut = 127.0f;
    float scale = max_span > 0.0f ? max_span / max_lut : 1.0f;
    float inv_scale;
    if (scale >= FLT_MIN) inv_scale = 1.0f / scale; else { scale = 1.0f; inv_scale = 1.0f; }
    for (size_t g = 0; g < G; g++) {
        for (int sub = 0; sub < 2; sub++) {
            float m = mins[g * 2 + (size_t)sub];
            for (int i = 0; i < 16; i++) {
                size_t j = g * 32 + (size_t)sub * 16 + (size_t)i;
                lut[j] = (uint8_t)clampf(roundf((fv[j] - m) * inv_scale), 0.0f, max_lut);
            }
        }
    }
    *scale_out = scale; *bias_out = bias;
    free(fv); free(mins);
}

/* search.rs:2806-2846 build_permute_dot */
void tvo_build_permute_dot(const float *q, const float *centroids, int dim,
                           int8_t levels[16], int8_t *weights, int32_t *zero, float *scale_out) {
    size_t G = (size_t)dim / 2;
    float cmax = 0.0f;
    for (int i = 0; i < 16; i++) { float v = fabsf(centroids[i]); if (v > cmax) cmax = v; }
    float cs = cmax > 0.0f ? cmax / 127.0f : 1.0f;
    for (int i = 0; i < 16; i++) levels[i] = (int8_t)clampf(roundf(centroids[i] / cs), -127.0f, 127.0f);
    float qmax = 0.0f;
    for (int d = 0; d < dim; d++) { float v = fabsf(q[d]); if (v > qmax) qmax = v; }
    float qs = qmax / 127.0f, inv_qs;
    if (qs >= FLT_MIN) inv_qs = 1.0f / qs; else { qs = 1.0f; inv_qs = 1.0f; }
    int32_t wsum = 0;
    for (size_t g = 0; g < G; g++) {
        size_t q4 = g / 4, j = g % 4;
        int8_t lo = (int8_t)clampf(roundf(q[2 * g + 1] * inv_qs), -127.0f, 127.0f);
        int8_t hi = (int8_t)clampf(roundf(q[2 * g] * inv_qs), -127.0f, 127.0f);
        weights[q4 * 8 + j] = lo;
        weights[q4 * 8 + 4 + j] = hi;
        wsum += (int32_t)lo + (int32_t)hi;
    }
    *zero = -128 * wsum;
    *scale_out = cs * qs;
}

/* search.rs:3154-3186 calibrate_queries, one row */
void tvo_calibrate_query(const float *q_rot, const float *shift, const float *scale_tq, int dim,
                         float *q_cal, float *bias_corr) {
    if (!shift || !scale_tq) {
        memcpy(q_cal, q_rot, sizeof(float) * (size_t)dim);
        *bias_corr = 0.0f;
        return;
    }
    double bc = 0.0;
    for (int d = 0; d < dim; d++) {
        q_cal[d] = q_rot[d] / scale_tq[d];
        bc -= (double)q_rot[d] * (double)shift[d];
    }
    *bias_corr = (float)bc;
}

/* ======================================================================= */
/* Search                                                                   */
/* ======================================================================= */

/* lib.rs:1363-1380 + encode.rs:76-83: first value with !(|x| < 1e16) */
int tvo_validate_queries(const float *queries, size_t len, int dim, size_t *bad_index) {
    if (dim <= 0 || len % (size_t)dim != 0) return TVO_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM;
    for (size_t i = 0; i < len; i++) {
        if (!(fabsf(queries[i]) < 1e16f)) { if (bad_index) *bad_index = i; return TVO_ERR_INVALID_QUERY_VALUE; }
    }
    return TVO_OK;
}

/* lib.rs:1435-1456 */
size_t tvo_pack_mask(const uint8_t *mask_bools, size_t n, uint64_t *words_out) {
    size_t n_words = (n + 63) / 64, allowed = 0;
    for (size_t w = 0; w < n_words; w++) {
        uint64_t word = 0;
        for (size_t bit = 0; bit < 64 && w * 64 + bit < n; bit++)
            word |= (uint64_t)(mask_bools[w * 64 + bit] != 0) << bit;
        allowed += (size_t)__builtin_popcountll(word);
        words_out[w] = word;
    }
    return allowed;
}

typedef struct {
    /* Mode L */
    uint8_t *lut; float l_scale, l_bias;
    /* Mode P: per-group weights split by nibble (w_hi[g] = dim 2g, w_lo[g] = dim 2g+1) */
    int8_t *w_hi, *w_lo; int8_t levels[16]; float p_scale, p_bias;
} query_tables;

/* search.rs:244-252 rescan_min */
static void rescan_min(const float *hs, const uint64_t *hi, size_t k, float *mn, size_t *mi_out) {
    size_t mi = 0;
    for (size_t h = 1; h < k; h++)
        if (hs[h] < hs[mi] || (hs[h] == hs[mi] && hi[h] > hi[mi])) mi = h;
    *mn = hs[mi]; *mi_out = mi;
}

typedef struct { float s; uint64_t i; } pair_t;
/* search.rs:4285-4289 (score desc by partial_cmp, then index asc) */
static int cmp_pair(const void *a, const void *b) {
    const pair_t *x = (const pair_t *)a, *y = (const pair_t *)b;
    if (x->s > y->s) return -1;
    if (x->s < y->s) return 1;
    return (x->i > y->i) - (x->i < y->i);
}

/* Integer accumulator + float epilogue of one (query, vector) pair. */
static inline float score_one(int mode, const query_tables *t, const uint8_t *seq, size_t G,
                              size_t b, size_t lane, float vec_scale, int32_t *acc_out) {
    const uint8_t *base = seq + b * G * TVO_BLOCK + lane;
    if (mode == TVO_MODE_P) {
        /* search.rs:1467-1512 net effect: exact signed dot (the +128 bias and the
         * `zero` seed cancel); epilogue search.rs:1519-1524 */
        int32_t acc = 0;
        for (size_t g = 0; g < G; g++) {
            unsigned byte = base[g * TVO_BLOCK];
            acc += (int32_t)t->w_hi[g] * (int32_t)t->levels[byte >> 4] +
                   (int32_t)t->w_lo[g] * (int32_t)t->levels[byte & 15];
        }
        *acc_out = acc;
        return fmaf((float)acc, t->p_scale, t->p_bias) * vec_scale;
    }
    if (mode == TVO_MODE_L_SCALAR) { /* search.rs:3113-3128 */
        float s = t->l_bias; uint32_t acc = 0;
        for (size_t g = 0; g < G; g++) {
            unsigned byte = base[g * TVO_BLOCK];
            uint8_t a = t->lut[g * 32 + (byte >> 4)], c = t->lut[g * 32 + 16 + (byte & 15)];
            s += t->l_scale * (float)a;
            s += t->l_scale * (float)c;
            acc += (uint32_t)a + (uint32_t)c;
        }
        *acc_out = (int32_t)acc;
        return s * vec_scale;
    }
    if (mode == TVO_MODE_L_CLASSIC) { /* search.rs:516-582, 1571-1600 */
        float fa = t->l_bias; uint32_t total = 0;
        for (size_t g0 = 0; g0 < G; g0 += TVO_FLUSH_EVERY) {
            size_t g1 = g0 + TVO_FLUSH_EVERY < G ? g0 + TVO_FLUSH_EVERY : G;
            uint32_t part = 0;
            for (size_t g = g0; g < g1; g++) {
                unsigned byte = base[g * TVO_BLOCK];
                part += (uint32_t)t->lut[g * 32 + (byte >> 4)] + (uint32_t)t->lut[g * 32 + 16 + (byte & 15)];
            }
            fa = fmaf(t->l_scale, (float)part, fa);
            total += part;
        }
        *acc_out = (int32_t)total;
        return fa * vec_scale;
    }
    /* TVO_MODE_L_U32: search.rs:1174-1177 */
    uint32_t acc = 0;
    for (size_t g = 0; g < G; g++) {
        unsigned byte = base[g * TVO_BLOCK];
        acc += (uint32_t)t->lut[g * 32 + (byte >> 4)] + (uint32_t)t->lut[g * 32 + 16 + (byte & 15)];
    }
    *acc_out = (int32_t)acc;
    return (((float)(int32_t)acc * t->l_scale) + t->l_bias) * vec_scale;
}

int tvo_search(int mode, const float *queries, size_t nq, const tvo_rotation *rot,
               const uint8_t *seq, const float *centroids, const float *vec_scales,
               const float *tq_shift, const float *tq_scale,
               int bits, int dim, size_t n, size_t k, const uint64_t *mask,
               float *out_scores, int64_t *out_indices, size_t *out_k_eff,
               int32_t *acc_dump, float *score_dump, int n_threads) {
    if (mode == TVO_MODE_AUTO) mode = bits == 4 ? TVO_MODE_P : TVO_MODE_L_U32;
    if (mode == TVO_MODE_P && bits != 4) return TVO_ERR_BAD_ARGUMENT;
    size_t G = tvo_n_byte_groups(bits, dim);
    size_t n_blocks = (n + TVO_BLOCK - 1) / TVO_BLOCK;
    /* search.rs:3222-3229 */
    size_t n_allowed = n;
    if (mask) {
        n_allowed = 0;
        for (size_t w = 0; w < (n + 63) / 64; w++) n_allowed += (size_t)__builtin_popcountll(mask[w]);
    }
    if (k > n_allowed) k = n_allowed;
    if (k > n) k = n;
    *out_k_eff = k;
    if (k == 0 || nq == 0) return TVO_OK;
    (void)n_threads;
    int err = 0;
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads > 1 ? n_threads : 1)
    for (long long qi = 0; qi < (long long)nq; qi++) {
        float *q_rot = (float *)malloc(sizeof(float) * (size_t)dim);
        float *q_cal = (float *)malloc(sizeof(float) * (size_t)dim);
        memcpy(q_rot, queries + (size_t)qi * dim, sizeof(float) * (size_t)dim);
        tvo_rotation_apply(rot, q_rot);                      /* search.rs:3237-3242 */
        float bias_corr;
        tvo_calibrate_query(q_rot, tq_shift, tq_scale, dim, q_cal, &bias_corr); /* :3251 */
        query_tables t; memset(&t, 0, sizeof t);
        if (mode == TVO_MODE_P) {
            int8_t *w = (int8_t *)malloc((size_t)dim);
            int32_t zero;
            tvo_build_permute_dot(q_cal, centroids, dim, t.levels, w, &zero, &t.p_scale);
            t.p_bias = 0.0f + bias_corr;                     /* search.rs:3262-3266 */
            t.w_hi = (int8_t *)malloc(G); t.w_lo = (int8_t *)malloc(G);
            for (size_t g = 0; g < G; g++) {
                t.w_lo[g] = w[(g / 4) * 8 + g % 4];
                t.w_hi[g] = w[(g / 4) * 8 + 4 + g % 4];
            }
            free(w);
        } else {
            t.lut = (uint8_t *)malloc(G * 32);
            tvo_build_lut(q_cal, centroids, bits, dim, t.lut, &t.l_scale, &t.l_bias);
            t.l_bias += bias_corr;                           /* search.rs:3261 */
        }
        pair_t *pairs;
        size_t np = 0;
        int use_heap = k <= 1024;
        float *hs = NULL; uint64_t *hi = NULL; size_t hsz = 0, hmi = 0; float hmin = -INFINITY;
        if (use_heap) {
            hs = (float *)malloc(sizeof(float) * k); hi = (uint64_t *)malloc(sizeof(uint64_t) * k);
            pairs = (pair_t *)malloc(sizeof(pair_t) * k);
        } else {
            pairs = (pair_t *)malloc(sizeof(pair_t) * n_allowed);
        }
        for (size_t b = 0; b < n_blocks; b++) {
            size_t base_vec = b * TVO_BLOCK;
            /* search.rs:3015-3029 block_has_allowed */
            if (mask && (((mask[base_vec >> 6] >> (base_vec & 63)) & 0xFFFFFFFFull) == 0)) {
                if (acc_dump || score_dump)
                    for (size_t lane = 0; lane < TVO_BLOCK && base_vec + lane < n; lane++) {
                        int32_t acc; float s = score_one(mode, &t, seq, G, b, lane, vec_scales[base_vec + lane], &acc);
                        if (acc_dump) acc_dump[(size_t)qi * n + base_vec + lane] = acc;
                        if (score_dump) score_dump[(size_t)qi * n + base_vec + lane] = s;
                    }
                continue;
            }
            for (size_t lane = 0; lane < TVO_BLOCK; lane++) {
                size_t vi = base_vec + lane;
                if (vi >= n) break;
                int allowed = !mask || ((mask[vi >> 6] >> (vi & 63)) & 1);
                if (!allowed && !acc_dump && !score_dump) continue;
                int32_t acc;
                float score = score_one(mode, &t, seq, G, b, lane, vec_scales[vi], &acc);
                if (acc_dump) acc_dump[(size_t)qi * n + vi] = acc;
                if (score_dump) score_dump[(size_t)qi * n + vi] = score;
                if (!allowed) continue;
                if (use_heap) { /* search.rs:3130-3144 */
                    if (hsz < k) {
                        hs[hsz] = score; hi[hsz] = vi; hsz++;
                        if (hsz == k) rescan_min(hs, hi, k, &hmin, &hmi);
                    } else if (score > hmin) {
                        hs[hmi] = score; hi[hmi] = vi;
                        rescan_min(hs, hi, k, &hmin, &hmi);
                    }
                } else {
                    pairs[np].s = score; pairs[np].i = vi; np++;
                }
            }
        }
        if (use_heap) { for (size_t j = 0; j < hsz; j++) { pairs[j].s = hs[j]; pairs[j].i = hi[j]; } np = hsz; }
        qsort(pairs, np, sizeof(pair_t), cmp_pair);          /* search.rs:4285-4290 */
        if (np < k) {
#pragma omp atomic write
            err = 1;
        }
        for (size_t j = 0; j < k && j < np; j++) {
            out_scores[(size_t)qi * k + j] = pairs[j].s;
            out_indices[(size_t)qi * k + j] = (int64_t)pairs[j].i;
        }
        free(pairs); free(hs); free(hi);
        free(t.lut); free(t.w_hi); free(t.w_lo);
        free(q_rot); free(q_cal);
    }
    return err ? TVO_ERR_BAD_ARGUMENT : TVO_OK;
}

/* ======================================================================= */
/* Throughput-oriented variant for the CPU baseline: same results as        */
/* tvo_search in modes P and L_U32 (tests compare them), organised like the */
/* reference's batch path (search.rs:4005-4050): block ranges are split     */
/* across threads, each block's codes are decoded once and reused by every  */
/* query, per-range heaps are merged by (score desc, slot asc).             */
/* ======================================================================= */

typedef struct {
    float *hs; uint64_t *hi; size_t sz, mi; float mn;
} heap_t;

static inline void heap_push(heap_t *h, size_t k, float score, uint64_t vi) {
    if (h->sz < k) {
        h->hs[h->sz] = score; h->hi[h->sz] = vi; h->sz++;
        if (h->sz == k) rescan_min(h->hs, h->hi, k, &h->mn, &h->mi);
    } else if (score > h->mn) {
        h->hs[h->mi] = score; h->hi[h->mi] = vi;
        rescan_min(h->hs, h->hi, k, &h->mn, &h->mi);
    }
}

__attribute__((target_clones("arch=skylake-avx512", "avx2", "default")))
int32_t tvo_dot_i8(const int8_t *a, const int8_t *b, int n) {
    int32_t s = 0;
    for (int i = 0; i < n; i++) s += (int32_t)a[i] * (int32_t)b[i];
    return s;
}

int tvo_search_fast(const float *queries, size_t nq, const tvo_rotation *rot,
                    const uint8_t *seq, const float *centroids, const float *vec_scales,
                    int bits, int dim, size_t n, size_t k, const uint64_t *mask,
                    float *out_scores, int64_t *out_indices, size_t *out_k_eff, int n_threads) {
    size_t G = tvo_n_byte_groups(bits, dim);
    size_t n_blocks = (n + TVO_BLOCK - 1) / TVO_BLOCK;
    size_t n_allowed = n;
    if (mask) {
        n_allowed = 0;
        for (size_t w = 0; w < (n + 63) / 64; w++) n_allowed += (size_t)__builtin_popcountll(mask[w]);
    }
    if (k > n_allowed) k = n_allowed;
    if (k > n) k = n;
    *out_k_eff = k;
    if (k == 0 || nq == 0) return TVO_OK;
    if (n_threads < 1) n_threads = 1;
    const int mode_p = bits == 4;
    /* per-query tables */
    int8_t *W = NULL; uint8_t *LUT = NULL; int8_t levels[16];
    float *qscale = (float *)malloc(sizeof(float) * nq), *qbias = (float *)malloc(sizeof(float) * nq);
    if (mode_p) W = (int8_t *)malloc(nq * (size_t)dim); else LUT = (uint8_t *)malloc(nq * G * 32);
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long long qi = 0; qi < (long long)nq; qi++) {
        float *q_rot = (float *)malloc(sizeof(float) * (size_t)dim);
        memcpy(q_rot, queries + (size_t)qi * dim, sizeof(float) * (size_t)dim);
        tvo_rotation_apply(rot, q_rot);
        if (mode_p) {
            int8_t *w = (int8_t *)malloc((size_t)dim); int32_t zero; int8_t lv[16];
            tvo_build_permute_dot(q_rot, centroids, dim, lv, w, &zero, &qscale[qi]);
            if (qi == 0) memcpy(levels, lv, 16);
            qbias[qi] = 0.0f;
            int8_t *dst = W + (size_t)qi * dim;      /* per-dimension order */
            for (size_t g = 0; g < G; g++) {
                dst[2 * g + 1] = w[(g / 4) * 8 + g % 4];
                dst[2 * g] = w[(g / 4) * 8 + 4 + g % 4];
            }
            free(w);
        } else {
            tvo_build_lut(q_rot, centroids, bits, dim, LUT + (size_t)qi * G * 32, &qscale[qi], &qbias[qi]);
        }
        free(q_rot);
    }
    if (mode_p && nq > 0) { /* levels are query independent; make sure thread 0's copy is visible */
        float cmax = 0.0f;
        for (int i = 0; i < 16; i++) { float v = fabsf(centroids[i]); if (v > cmax) cmax = v; }
        float cs = cmax > 0.0f ? cmax / 127.0f : 1.0f;
        for (int i = 0; i < 16; i++) levels[i] = (int8_t)clampf(roundf(centroids[i] / cs), -127.0f, 127.0f);
    }
    /* block ranges: even block counts so ranges start on mask-word boundaries (search.rs:3038) */
    size_t n_ranges = (size_t)n_threads * 4;
    size_t stride = (n_blocks + n_ranges - 1) / n_ranges;
    if (stride < 2) stride = 2;
    stride += stride & 1;
    n_ranges = (n_blocks + stride - 1) / stride;
    float *all_s = (float *)malloc(sizeof(float) * n_ranges * nq * k);
    uint64_t *all_i = (uint64_t *)malloc(sizeof(uint64_t) * n_ranges * nq * k);
    size_t *all_sz = (size_t *)calloc(n_ranges * nq, sizeof(size_t));
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
    for (long long r = 0; r < (long long)n_ranges; r++) {
        size_t b0 = (size_t)r * stride, b1 = b0 + stride < n_blocks ? b0 + stride : n_blocks;
        heap_t *heaps = (heap_t *)malloc(sizeof(heap_t) * nq);
        for (size_t qi = 0; qi < nq; qi++) {
            heaps[qi].hs = all_s + ((size_t)r * nq + qi) * k;
            heaps[qi].hi = all_i + ((size_t)r * nq + qi) * k;
            heaps[qi].sz = 0; heaps[qi].mi = 0; heaps[qi].mn = -INFINITY;
        }
        int8_t *dec = mode_p ? (int8_t *)malloc((size_t)TVO_BLOCK * (size_t)dim) : NULL;
        for (size_t b = b0; b < b1; b++) {
            size_t base_vec = b * TVO_BLOCK;
            uint32_t mw = 0xFFFFFFFFu;
            if (mask) { mw = (uint32_t)(mask[base_vec >> 6] >> (base_vec & 63)); if (!mw) continue; }
            size_t lanes = n - base_vec < TVO_BLOCK ? n - base_vec : TVO_BLOCK;
            const uint8_t *blk = seq + b * G * TVO_BLOCK;
            if (mode_p) {
                for (size_t g = 0; g < G; g++)
                    for (size_t l = 0; l < lanes; l++) {
                        unsigned byte = blk[g * TVO_BLOCK + l];
                        dec[l * (size_t)dim + 2 * g] = levels[byte >> 4];
                        dec[l * (size_t)dim + 2 * g + 1] = levels[byte & 15];
                    }
                for (size_t qi = 0; qi < nq; qi++) {
                    const int8_t *w = W + qi * (size_t)dim;
                    for (size_t l = 0; l < lanes; l++) {
                        if (!((mw >> l) & 1)) continue;
                        int32_t acc = tvo_dot_i8(w, dec + l * (size_t)dim, dim);
                        float score = fmaf((float)acc, qscale[qi], qbias[qi]) * vec_scales[base_vec + l];
                        heap_push(&heaps[qi], k, score, base_vec + l);
                    }
                }
            } else {
                for (size_t qi = 0; qi < nq; qi++) {
                    const uint8_t *lut = LUT + qi * G * 32;
                    uint32_t acc[TVO_BLOCK] = {0};
                    for (size_t g = 0; g < G; g++) {
                        const uint8_t *row = lut + g * 32;
                        const uint8_t *cb = blk + g * TVO_BLOCK;
                        for (size_t l = 0; l < TVO_BLOCK; l++) acc[l] += (uint32_t)row[cb[l] >> 4] + (uint32_t)row[16 + (cb[l] & 15)];
                    }
                    for (size_t l = 0; l < lanes; l++) {
                        if (!((mw >> l) & 1)) continue;
                        float score = (((float)(int32_t)acc[l] * qscale[qi]) + qbias[qi]) * vec_scales[base_vec + l];
                        heap_push(&heaps[qi], k, score, base_vec + l);
                    }
                }
            }
        }
        for (size_t qi = 0; qi < nq; qi++) all_sz[(size_t)r * nq + qi] = heaps[qi].sz;
        free(dec); free(heaps);
    }
    int err = 0;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long long qi = 0; qi < (long long)nq; qi++) {
        pair_t *pairs = (pair_t *)malloc(sizeof(pair_t) * n_ranges * k);
        size_t np = 0;
        for (size_t r = 0; r < n_ranges; r++) {
            size_t sz = all_sz[r * nq + (size_t)qi];
            for (size_t j = 0; j < sz; j++) {
                pairs[np].s = all_s[(r * nq + (size_t)qi) * k + j];
                pairs[np].i = all_i[(r * nq + (size_t)qi) * k + j];
                np++;
            }
        }
        qsort(pairs, np, sizeof(pair_t), cmp_pair);          /* search.rs:4279-4298 */
        if (np < k) {
#pragma omp atomic write
            err = 1;
        }
        for (size_t j = 0; j < k && j < np; j++) {
            out_scores[(size_t)qi * k + j] = pairs[j].s;
            out_indices[(size_t)qi * k + j] = (int64_t)pairs[j].i;
        }
        free(pairs);
    }
    free(all_s); free(all_i); free(all_sz); free(qscale); free(qbias); free(W); free(LUT);
    return err ? TVO_ERR_BAD_ARGUMENT : TVO_OK;
}

/* ======================================================================= */
/* The reference's production kernel for 4-bit on AVX-512 VNNI hosts:        */
/* search_multi_query_permute_dot (search.rs:1392-1567) over the             */
/* vector-major layout (pack.rs:1269-1271, :1347-1358), eight queries per    */
/* pass over a block.  Same integers and floats as tvo_search mode P (tests  */
/* compare them); this is what the CPU-baseline timing runs when the host    */
/* has the instructions, so that the baseline runs the reference's           */
/* algorithm at the reference's speed.                                       */
/* ======================================================================= */

/* pack.rs:1347-1358 vector_major_chunk over every unit of 4 byte-groups x 32 vectors:
 * byte of (group 4*q4 + j, vector v) moves to q4*128 + (v/16)*64 + (v%16)*4 + j.
 * dim*bits/8 must be a multiple of 4 (pack.rs:1260-1263).  Out of place. */
int tvo_seq_to_vector_major(const uint8_t *seq, size_t n, int bits, int dim, uint8_t *vm) {
    size_t G = tvo_n_byte_groups(bits, dim);
    if (G % 4 != 0) return TVO_ERR_BAD_ARGUMENT;
    size_t n_units = (n + TVO_BLOCK - 1) / TVO_BLOCK * (G / 4);
    for (size_t u = 0; u < n_units; u++) {
        const uint8_t *src = seq + u * 128;
        uint8_t *dst = vm + u * 128;
        for (int j = 0; j < 4; j++)
            for (int v = 0; v < TVO_BLOCK; v++) dst[(v / 16) * 64 + (v % 16) * 4 + j] = src[j * TVO_BLOCK + v];
    }
    return TVO_OK;
}

#if defined(__x86_64__)
#include <immintrin.h>

int tvo_have_vnni(void) {
    __builtin_cpu_init();
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vnni");
}

#define TVO_NQ 8

/* One block range, up to eight queries: search.rs:1417-1545.  w8: the queries' weights in the
 * reference's quad layout ([q4*8 + j] = low-nibble weight of group 4*q4 + j, [q4*8 + 4 + j] = high). */
__attribute__((target("avx2,fma,avx512f,avx512bw,avx512vnni"), always_inline))
static inline void scan_range_vnni_n(const uint8_t *vm, size_t G, size_t b0, size_t b1, size_t n,
                                     const int8_t *const *w8, const int32_t *zero, const float *qscale,
                                     const float *qbias, const int nqm, const int8_t *levels16,
                                     const float *vec_scales, const uint64_t *mask, heap_t *heaps, size_t k) {
    const __m512i m0f = _mm512_set1_epi8(0x0F);
    const size_t quads = G / 4, block_bytes = G * TVO_BLOCK;
    /* +128 puts the signed levels into vpdpbusd's unsigned operand; `zero` cancels it (search.rs:1426-1429) */
    const __m512i levels = _mm512_xor_si512(_mm512_broadcast_i32x4(_mm_loadu_si128((const __m128i *)levels16)),
                                            _mm512_set1_epi8((char)0x80));
    for (size_t b = b0; b < b1; b++) {
        const size_t base_vec = b * TVO_BLOCK;
        uint32_t mw = 0xFFFFFFFFu;
        if (mask) { mw = (uint32_t)(mask[base_vec >> 6] >> (base_vec & 63)); if (!mw) continue; }   /* search.rs:3015-3029 */
        const uint8_t *blk = vm + b * block_bytes;
        __m512i acc[TVO_NQ][2];
        for (int qi = 0; qi < nqm; qi++) { acc[qi][0] = _mm512_set1_epi32(zero[qi]); acc[qi][1] = acc[qi][0]; }
        for (size_t q4 = 0; q4 < quads; q4++) {
            for (int h = 0; h < 2; h++) {
                const uint8_t *p = blk + q4 * 128 + (size_t)h * 64;
                _mm_prefetch((const char *)(p + 32 * 128), _MM_HINT_T0);
                const __m512i c = _mm512_loadu_si512((const void *)p);
                const __m512i vlo = _mm512_shuffle_epi8(levels, _mm512_and_si512(c, m0f));
                const __m512i vhi = _mm512_shuffle_epi8(levels, _mm512_and_si512(_mm512_srli_epi16(c, 4), m0f));
                for (int qi = 0; qi < nqm; qi++) {
                    int32_t wl, wh;
                    memcpy(&wl, w8[qi] + q4 * 8, 4);
                    memcpy(&wh, w8[qi] + q4 * 8 + 4, 4);
                    acc[qi][h] = _mm512_dpbusd_epi32(acc[qi][h], vlo, _mm512_set1_epi32(wl));
                    acc[qi][h] = _mm512_dpbusd_epi32(acc[qi][h], vhi, _mm512_set1_epi32(wh));
                }
            }
        }
        const size_t lanes = n - base_vec < TVO_BLOCK ? n - base_vec : TVO_BLOCK;
        const int full = lanes == TVO_BLOCK;
        float vsb[TVO_BLOCK];
        for (size_t l = 0; l < TVO_BLOCK; l++) vsb[l] = l < lanes ? vec_scales[base_vec + l] : 0.0f;
        for (int qi = 0; qi < nqm; qi++) {
            /* search.rs:1519-1524: fma(f32(acc), scale, bias), then the row scale (:1793-1794) */
            const __m512 vs = _mm512_set1_ps(qscale[qi]), vb = _mm512_set1_ps(qbias[qi]);
            const __m512 s0 = _mm512_mul_ps(_mm512_fmadd_ps(_mm512_cvtepi32_ps(acc[qi][0]), vs, vb), _mm512_loadu_ps(vsb));
            const __m512 s1 = _mm512_mul_ps(_mm512_fmadd_ps(_mm512_cvtepi32_ps(acc[qi][1]), vs, vb), _mm512_loadu_ps(vsb + 16));
            heap_t *hp = &heaps[qi];
            if (hp->sz >= k && full) {   /* search.rs:1792-1800: nothing in the block beats the heap's minimum */
                const __m512 thr = _mm512_set1_ps(hp->mn);
                if ((_mm512_cmp_ps_mask(s0, thr, _CMP_GT_OQ) | _mm512_cmp_ps_mask(s1, thr, _CMP_GT_OQ)) == 0) continue;
            }
            float out[TVO_BLOCK];
            _mm512_storeu_ps(out, s0);
            _mm512_storeu_ps(out + 16, s1);
            for (size_t l = 0; l < lanes; l++) {
                if (!((mw >> l) & 1)) continue;
                heap_push(hp, k, out[l], base_vec + l);
            }
        }
    }
}

/* The query count is a compile-time constant in each instance (the reference's const generic NQ),
 * so the accumulators of all eight queries live in registers. */
__attribute__((target("avx2,fma,avx512f,avx512bw,avx512vnni")))
static void scan_range_vnni(const uint8_t *vm, size_t G, size_t b0, size_t b1, size_t n,
                            const int8_t *const *w8, const int32_t *zero, const float *qscale,
                            const float *qbias, int nqm, const int8_t *levels16,
                            const float *vec_scales, const uint64_t *mask, heap_t *heaps, size_t k) {
#define TVO_CASE(N) case N: scan_range_vnni_n(vm, G, b0, b1, n, w8, zero, qscale, qbias, N, levels16, vec_scales, mask, heaps, k); break
    switch (nqm) {
        TVO_CASE(1); TVO_CASE(2); TVO_CASE(3); TVO_CASE(4); TVO_CASE(5); TVO_CASE(6); TVO_CASE(7); TVO_CASE(8);
        default: break;
    }
#undef TVO_CASE
}
#else
int tvo_have_vnni(void) { return 0; }
#endif

/* search::search for 4-bit indexes held in the vector-major layout: block ranges over threads,
 * inside a range eight queries per pass (search.rs:3996-4050), per-range heaps merged by
 * (score desc, slot asc) (search.rs:4279-4298).  Uncalibrated indexes, k <= 1024.  Returns
 * TVO_ERR_BAD_ARGUMENT when the host lacks AVX-512 VNNI. */
int tvo_search_vnni(const float *queries, size_t nq, const tvo_rotation *rot,
                    const uint8_t *vm_codes, const float *centroids, const float *vec_scales,
                    int dim, size_t n, size_t k, const uint64_t *mask,
                    float *out_scores, int64_t *out_indices, size_t *out_k_eff, int n_threads) {
#if defined(__x86_64__)
    if (!tvo_have_vnni()) return TVO_ERR_BAD_ARGUMENT;
    const size_t G = (size_t)dim / 2;
    if (G % 4 != 0) return TVO_ERR_BAD_ARGUMENT;
    const size_t n_blocks = (n + TVO_BLOCK - 1) / TVO_BLOCK;
    size_t n_allowed = n;
    if (mask) {
        n_allowed = 0;
        for (size_t w = 0; w < (n + 63) / 64; w++) n_allowed += (size_t)__builtin_popcountll(mask[w]);
    }
    if (k > n_allowed) k = n_allowed;
    if (k > n) k = n;
    *out_k_eff = k;
    if (k == 0 || nq == 0) return TVO_OK;
    if (n_threads < 1) n_threads = 1;
    int8_t *W = (int8_t *)malloc(nq * (size_t)dim);
    int32_t *zero = (int32_t *)malloc(sizeof(int32_t) * nq);
    float *qscale = (float *)malloc(sizeof(float) * nq), *qbias = (float *)calloc(nq, sizeof(float));
    int8_t levels[16];
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long long qi = 0; qi < (long long)nq; qi++) {
        float *q_rot = (float *)malloc(sizeof(float) * (size_t)dim);
        memcpy(q_rot, queries + (size_t)qi * dim, sizeof(float) * (size_t)dim);
        tvo_rotation_apply(rot, q_rot);
        int8_t lv[16];
        tvo_build_permute_dot(q_rot, centroids, dim, lv, W + (size_t)qi * dim, &zero[qi], &qscale[qi]);
        free(q_rot);
    }
    {
        float cmax = 0.0f;
        for (int i = 0; i < 16; i++) { float v = fabsf(centroids[i]); if (v > cmax) cmax = v; }
        float cs = cmax > 0.0f ? cmax / 127.0f : 1.0f;
        for (int i = 0; i < 16; i++) levels[i] = (int8_t)clampf(roundf(centroids[i] / cs), -127.0f, 127.0f);
    }
    /* Tiles = query groups of eight x block ranges, as the reference's batch dispatch cuts them
     * (search.rs:125-144 n_block_ranges with TILES_PER_THREAD = 32 :178 and MIN_TILE_BLOCKS_X86 =
     * 3072 :226, :265-278 range_cap_for_k, :284-295 smooth_tile_count; a mask keeps one range,
     * :111-113), drawn block-range-major by the pool (search.rs:4031-4046). */
    const size_t n_groups = (nq + TVO_NQ - 1) / TVO_NQ;
    size_t n_ranges = 1;
    if (n_threads > 1 && !mask) {
        n_ranges = ((size_t)n_threads * 32 + n_groups - 1) / n_groups;
        const size_t by_blocks = (n_blocks + 3071) / 3072;
        size_t by_k = (n + 512 * k - 1) / (512 * k);
        if (by_k < 1) by_k = 1;
        if (n_ranges > by_blocks) n_ranges = by_blocks;
        if (n_ranges > by_k) n_ranges = by_k;
        if (n_ranges < 1) n_ranges = 1;
        const size_t tiles = n_groups * n_ranges;
        if (tiles > (size_t)n_threads && tiles < 2 * (size_t)n_threads) {
            n_ranges = (size_t)n_threads / n_groups;
            if (n_ranges < 1) n_ranges = 1;
        }
    }
    size_t stride = (n_blocks + n_ranges - 1) / n_ranges;
    if (stride < 1) stride = 1;
    stride += stride & 1;                   /* ranges start on mask-word boundaries (search.rs:3038) */
    n_ranges = (n_blocks + stride - 1) / stride;
    float *all_s = (float *)malloc(sizeof(float) * n_ranges * nq * k);
    uint64_t *all_i = (uint64_t *)malloc(sizeof(uint64_t) * n_ranges * nq * k);
    size_t *all_sz = (size_t *)calloc(n_ranges * nq, sizeof(size_t));
    const long long n_tiles = (long long)(n_ranges * n_groups);
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
    for (long long t = 0; t < n_tiles; t++) {
        const size_t r = (size_t)t / n_groups, q0 = ((size_t)t % n_groups) * TVO_NQ;
        const size_t b0 = r * stride, b1 = b0 + stride < n_blocks ? b0 + stride : n_blocks;
        heap_t heaps[TVO_NQ];
        const int nqm = (int)(nq - q0 < TVO_NQ ? nq - q0 : TVO_NQ);
        const int8_t *w8[TVO_NQ];
        for (int j = 0; j < nqm; j++) {
            w8[j] = W + (q0 + (size_t)j) * (size_t)dim;
            heaps[j].hs = all_s + (r * nq + q0 + (size_t)j) * k;
            heaps[j].hi = all_i + (r * nq + q0 + (size_t)j) * k;
            heaps[j].sz = 0; heaps[j].mi = 0; heaps[j].mn = -INFINITY;
        }
        scan_range_vnni(vm_codes, G, b0, b1, n, w8, zero + q0, qscale + q0, qbias + q0, nqm, levels,
                        vec_scales, mask, heaps, k);
        for (int j = 0; j < nqm; j++) all_sz[r * nq + q0 + (size_t)j] = heaps[j].sz;
    }
    int err = 0;
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long long qi = 0; qi < (long long)nq; qi++) {
        pair_t *pairs = (pair_t *)malloc(sizeof(pair_t) * n_ranges * k);
        size_t np = 0;
        for (size_t r = 0; r < n_ranges; r++) {
            size_t sz = all_sz[r * nq + (size_t)qi];
            for (size_t j = 0; j < sz; j++) {
                pairs[np].s = all_s[(r * nq + (size_t)qi) * k + j];
                pairs[np].i = all_i[(r * nq + (size_t)qi) * k + j];
                np++;
            }
        }
        qsort(pairs, np, sizeof(pair_t), cmp_pair);          /* search.rs:4279-4298 */
        if (np < k) {
#pragma omp atomic write
            err = 1;
        }
        for (size_t j = 0; j < k && j < np; j++) {
            out_scores[(size_t)qi * k + j] = pairs[j].s;
            out_indices[(size_t)qi * k + j] = (int64_t)pairs[j].i;
        }
        free(pairs);
    }
    free(all_s); free(all_i); free(all_sz); free(qscale); free(qbias); free(W); free(zero);
    return err ? TVO_ERR_BAD_ARGUMENT : TVO_OK;
#else
    (void)queries; (void)nq; (void)rot; (void)vm_codes; (void)centroids; (void)vec_scales; (void)dim; (void)n; (void)k;
    (void)mask; (void)out_scores; (void)out_indices; (void)out_k_eff; (void)n_threads;
    return TVO_ERR_BAD_ARGUMENT;
#endif
}

/* ======================================================================= */
/* Fixture helpers                                                          */
/* ======================================================================= */

/* tests/common/fingerprint.rs:80-90 lcg_vectors */
void tvo_lcg_vectors(size_t count, uint64_t seed, float *out) {
    uint64_t state = seed | 1;
    for (size_t i = 0; i < count; i++) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        out[i] = (float)((double)(uint32_t)(state >> 32) / 2147483648.0 - 1.0);
    }
}

/* tests/common/fingerprint.rs:58-66 */
uint64_t tvo_fnv1a(const uint8_t *bytes, size_t len) {
    uint64_t h = 0xcbf29ce484222325ull;
    for (size_t i = 0; i < len; i++) { h ^= bytes[i]; h *= 0x100000001b3ull; }
    return h;
}
