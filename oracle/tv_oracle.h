/*
 * tv_oracle.h -- CPU restatement of the turbovec search path (TEST INFRASTRUCTURE).
 *
 * This library is the checker that the HIP search path is compared against.
 * It is not part of the product: nothing under turbovec_amd/ links, loads or
 * calls it.  Only tests, the smoke check and the CPU-baseline leg of the
 * benchmark use it.
 *
 * Every function names the reference file:line it restates (paths relative to
 * the turbovec repository root, e.g. turbovec/src/search.rs:3206).
 *
 * Parity status per function (what pins it besides a line-by-line reading):
 *   tvo_rotation_*           pinned: golden f32 bit patterns dim 8/24/64 and the
 *                            dim-128 fold (tests/rotation_determinism.rs:75-96,
 *                            src/rotation.rs:1325); dims 1536/3072 end-to-end by
 *                            the encode fingerprint codes/scales hashes.
 *   tvo_codebook             pinned: FNV-1a-64 of boundaries/centroids for 8
 *                            (dim,bits) cells (tests/encode_fingerprint.rs:83-92).
 *                            Cells without a golden, (128,4) among them: an
 *                            independent Lloyd-Max (cell probabilities from scipy's
 *                            incomplete beta function, conditional means in closed
 *                            form, no quadrature) reproduces the golden hashes and
 *                            equals this function bit for bit in every cell.
 *   tvo_search_fast,         equality with tvo_search on the same inputs (tests).
 *   tvo_search_vnni
 *   tvo_fit_calibration,
 *   tvo_encode, tvo_norm     pinned: calibration/codes/scales hashes, 8 cells.
 *   tvo_repack_seq et al.    pinned: closed-form byte maps (src/pack.rs:964-1008).
 *   tvo_build_lut            pinned end to end at 4-bit through the parity fixture below
 *                            (any wrong entry, scale or bias moves one of its 600
 *                            floats); at 2, 3 and 4 bits every byte, the scale and the
 *                            bias equal an independent numpy float32 model.
 *   tvo_search  L_CLASSIC    pinned at 4-bit: the 3 x 200 float scores and ids of
 *                            benchmarks/hillclimb/data/parity_base_{x86,arm}.json are
 *                            reproduced bit for bit (base, after the warm appends,
 *                            after 500 swap-removes).
 *   tvo_build_permute_dot    pinned: slot map and zero identity (src/search.rs:4596);
 *                            every weight, level, zero and scale equal an independent
 *                            numpy float32 model over 360 queries (dims 128/1536/3072),
 *                            half-way values (round half away from zero) and the
 *                            +-127 ends included.
 *   tvo_calibrate_query      pinned: exact-rational model of the sequential f64 sum
 *                            (inputs chosen so that a float32 accumulator, an exactly
 *                            rounded sum, the reversed order and the opposite sign all
 *                            give another answer).
 *   tvo_search  mode P,      pinned: the reference holds no vector written by these
 *               L_U32,       kernels (the fixture above was written by the classic LUT
 *               L_SCALAR     kernel), so every float score is compared with an
 *                            exact-rational evaluation of its epilogue, each IEEE
 *                            operation rounded once (P: fma(f32(acc), scale, bias) *
 *                            row scale, |acc| > 2^24 included; L_U32: multiply, add,
 *                            multiply; L_SCALAR: two multiply-adds per group), on
 *                            TQ+-calibrated indexes so the bias is not zero and fused
 *                            and unfused forms differ; integers by brute force over
 *                            decoded codes; scores estimate true inner products to
 *                            quantisation noise (src/kernel_tests.rs:401-419).
 *                            All of this lives in tests/test_oracle_pins.py.
 */
#ifndef TV_ORACLE_H
#define TV_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TVO_BLOCK 32            /* turbovec/src/lib.rs:89  */
#define TVO_FLUSH_EVERY 256     /* turbovec/src/lib.rs:102 */
#define TVO_MAX_DIM 16384       /* turbovec/src/lib.rs:101 */

/* Scoring modes (which integer definition + float epilogue the scan uses). */
enum {
    TVO_MODE_AUTO = 0,      /* what a VNNI x86 host runs: P at 4-bit, L_U32 otherwise */
    TVO_MODE_L_SCALAR = 1,  /* search.rs:3077-3147 */
    TVO_MODE_L_CLASSIC = 2, /* search.rs:516-582 (u16 batches of 256 groups, fma flush) */
    TVO_MODE_L_U32 = 3,     /* search.rs:1174-1177 (u32 sum, mul then add) */
    TVO_MODE_P = 4          /* search.rs:1519-1524 (int8 dot, fma epilogue), 4-bit only */
};

/* Status codes shared with the product C ABI (same numeric values). */
enum {
    TVO_OK = 0,
    TVO_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM = 1,
    TVO_ERR_INVALID_QUERY_VALUE = 2,
    TVO_ERR_MASK_LENGTH_MISMATCH = 3,
    TVO_ERR_ALLOWLIST_EMPTY = 4,
    TVO_ERR_UNKNOWN_ID = 5,
    TVO_ERR_BAD_ARGUMENT = 6
};

/* ---- ChaCha8 stream (rand_chacha =0.3.1, not vendored in the reference) ---- */
typedef struct {
    uint32_t key[8];
    uint64_t counter;   /* block counter of the next refill */
    uint32_t buf[64];   /* four consecutive 16-word blocks */
    int index;          /* next unread word, 64 = exhausted */
} tvo_chacha8;
void tvo_chacha8_init(tvo_chacha8 *rng, const uint8_t seed[32]);
uint32_t tvo_chacha8_next_u32(tvo_chacha8 *rng);
uint64_t tvo_chacha8_next_u64(tvo_chacha8 *rng);

/* ---- Rotation (turbovec/src/rotation.rs:103-187, 265-320) ---- */
typedef struct {
    int dim;
    int block;
    float inv_sqrt_block;
    float *signs[2];
    uint32_t *perms[2];
} tvo_rotation;
tvo_rotation *tvo_rotation_new(int dim);
void tvo_rotation_free(tvo_rotation *r);
int tvo_rotation_block(const tvo_rotation *r);
const float *tvo_rotation_signs(const tvo_rotation *r, int round);
const uint32_t *tvo_rotation_perm(const tvo_rotation *r, int round);
/* rotation.rs:265 apply_with_scratch: row rotated in place. */
void tvo_rotation_apply(const tvo_rotation *r, float *row);
/* rotation.rs:218 apply_scaled_into: dst = rotate(src * inv). */
void tvo_rotation_apply_scaled(const tvo_rotation *r, const float *src, float inv, float *dst);

/* ---- Codebook (turbovec/src/codebook.rs:69-167) ---- */
double tvo_beta_cdf(double a, double x);  /* Beta(a,a).cdf(x), statrs =0.17.1 */
double tvo_beta_pdf(double a, double x);  /* Beta(a,a).pdf(x) */
/* boundaries[2^bits-1], centroids[2^bits]. */
int tvo_codebook(int bits, int dim, float *boundaries, float *centroids);

/* ---- Encode (turbovec/src/encode.rs) ---- */
float tvo_norm(const float *row, int dim);                          /* encode.rs:900-932 */
/* encode.rs:737-857; rotated rows are produced inside from raw vectors (encode.rs:470-481). */
void tvo_fit_calibration(const tvo_rotation *r, const float *vectors, size_t n, int dim,
                         const float *centroids, int n_levels, float *shift, float *scale);
/* encode.rs:510-548 + 560-664 + 1418-1476.  shift/scale_tq may be NULL (identity).
 * packed_out: n * bits * dim/8 bytes (bit-plane rows); scales_out: n floats. */
void tvo_encode(const tvo_rotation *r, const float *vectors, size_t n, int dim, int bits,
                const float *boundaries, const float *centroids,
                const float *shift, const float *scale_tq,
                uint8_t *packed_out, float *scales_out);

/* ---- Layouts (turbovec/src/pack.rs) ---- */
size_t tvo_n_byte_groups(int bits, int dim);                         /* pack.rs:252-257 */
size_t tvo_seq_len(size_t n, int bits, int dim);
void tvo_repack_seq(const uint8_t *packed, size_t n, int bits, int dim, uint8_t *seq_out); /* pack.rs:366 */
void tvo_seq_to_packed(const uint8_t *seq, size_t n, int bits, int dim, uint8_t *packed_out); /* pack.rs:375 */
/* lib.rs:2964-3003: move the last vector into slot idx, zero the vacated lane.
 * seq must hold the geometry for n vectors; returns the new count n-1. */
size_t tvo_swap_remove_seq(uint8_t *seq, float *scales, size_t n, int bits, int dim, size_t idx);

/* ---- Query preparation (turbovec/src/search.rs) ---- */
/* search.rs:2856-2994. lut: G*32 bytes ([sub-table for the HIGH nibble | LOW nibble] per group). */
void tvo_build_lut(const float *q_rot, const float *centroids, int bits, int dim,
                   uint8_t *lut, float *scale, float *bias);
/* search.rs:2806-2846. weights: dim bytes in the reference's quad layout. */
void tvo_build_permute_dot(const float *q_rot, const float *centroids, int dim,
                           int8_t levels[16], int8_t *weights, int32_t *zero, float *scale);
/* search.rs:3154-3186. shift/scale_tq NULL => copy and 0. */
void tvo_calibrate_query(const float *q_rot, const float *shift, const float *scale_tq, int dim,
                         float *q_cal, float *bias_corr);

/* ---- Search (turbovec/src/search.rs:3206-3353 restated over the seq-blocked layout) ----
 * queries: nq*dim raw floats.  mask_words: NULL or ceil(n/64) words.  k_eff =
 * min(k, n, popcount(mask)).  out_scores/out_indices: nq*k_eff entries, rows sorted
 * (score desc, slot asc).  acc_dump (optional): nq*n int32 integer accumulators
 * (mode P: signed dot; modes L: total u8 sum).  score_dump (optional): nq*n floats.
 * n_threads <= 1 runs single-threaded. */
int tvo_search(int mode, const float *queries, size_t nq, const tvo_rotation *rot,
               const uint8_t *seq_codes, const float *centroids, const float *vec_scales,
               const float *tq_shift, const float *tq_scale,
               int bits, int dim, size_t n, size_t k, const uint64_t *mask_words,
               float *out_scores, int64_t *out_indices, size_t *out_k_eff,
               int32_t *acc_dump, float *score_dump, int n_threads);

/* Same answer as tvo_search in the modes a VNNI host runs (P at 4-bit, L_U32
 * otherwise), uncalibrated indexes, k <= 1024; organised for throughput (block
 * ranges over threads, codes decoded once per block, per-range heaps merged as
 * search.rs:4279-4298 does).  This is what the CPU-baseline timing runs. */
int tvo_search_fast(const float *queries, size_t nq, const tvo_rotation *rot,
                    const uint8_t *seq_codes, const float *centroids, const float *vec_scales,
                    int bits, int dim, size_t n, size_t k, const uint64_t *mask_words,
                    float *out_scores, int64_t *out_indices, size_t *out_k_eff, int n_threads);

/* The reference's production path for 4-bit on an AVX-512 VNNI host (search.rs:1392-1567):
 * vpshufb level lookup + vpdpbusd over the vector-major layout (pack.rs:1269-1271), eight
 * queries per pass over a block.  tvo_seq_to_vector_major builds that layout (what the
 * reference keeps at rest, pack.rs:1347-1358); tvo_search_vnni answers exactly as tvo_search
 * mode P does (tests compare bit for bit) and returns TVO_ERR_BAD_ARGUMENT on a host without
 * the instructions (tvo_have_vnni() == 0).  Uncalibrated indexes, k <= 1024.  This is what the
 * CPU-baseline timing runs where it can. */
int tvo_have_vnni(void);
int tvo_seq_to_vector_major(const uint8_t *seq, size_t n, int bits, int dim, uint8_t *vm);
int tvo_search_vnni(const float *queries, size_t nq, const tvo_rotation *rot,
                    const uint8_t *vm_codes, const float *centroids, const float *vec_scales,
                    int dim, size_t n, size_t k, const uint64_t *mask_words,
                    float *out_scores, int64_t *out_indices, size_t *out_k_eff, int n_threads);

/* Caller-side checks that precede the seam (turbovec/src/lib.rs:1363-1380,
 * encode.rs:76-83): returns TVO_OK or the error; *bad_index = flat offset. */
int tvo_validate_queries(const float *queries, size_t len, int dim, size_t *bad_index);
/* lib.rs:1435-1456: bool bytes -> u64 words, returns popcount. */
size_t tvo_pack_mask(const uint8_t *mask_bools, size_t n, uint64_t *words_out);

/* ---- Test-fixture helpers restating the reference's own generators ---- */
/* tests/common/fingerprint.rs:80-90 */
void tvo_lcg_vectors(size_t count, uint64_t seed, float *out);
/* tests/common/fingerprint.rs:58-66 */
uint64_t tvo_fnv1a(const uint8_t *bytes, size_t len);

#ifdef __cplusplus
}
#endif
#endif
