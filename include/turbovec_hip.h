/*
 * turbovec_hip.h -- C ABI of the MI355X (gfx950) search path for turbovec.
 *
 * The library replaces ONE crate-internal function of the reference,
 *     search::search(...)                       turbovec/src/search.rs:3206-3221
 * whose only caller is
 *     TurboQuantIndex::try_search_with_mask     turbovec/src/lib.rs:1462-1477
 * plus the small amount of index state that function reads (codes, per-vector
 * scales, rotation tables, centroids, TQ+ calibration), kept resident in HBM.
 *
 * Conventions: every entry point returns a tv_status; nothing throws or aborts
 * across the boundary; all buffers are caller-owned host memory unless the name
 * ends in _dev; sizes are element counts.  Functions that mutate an index
 * (upload / append / swap_remove / set_*) need external exclusion, exactly as
 * the reference's `&mut self` methods do; tv_search* may be called from many
 * threads at once: the GPU serves one launch at a time, so calls that arrive
 * while the index is busy wait, and whoever gets the index next serves every
 * waiting tv_search (or tv_search_dev) call with the same k and the same mask
 * pointer together with its own, as one batch; each caller receives exactly the
 * rows a call of its own would have returned.  A process
 * that has used the library must not fork() and keep using it in the child.
 *
 * Device buffers (_dev entry points, device pointers): the library runs on a
 * stream of its own per index, not on the caller's.  Every device buffer handed
 * in must be complete -- the work that writes it finished, e.g. the producing
 * stream synchronised -- before the call, and must stay untouched until the call
 * returns; outputs are complete when the call returns (it synchronises its
 * stream before returning).
 */
#ifndef TURBOVEC_HIP_H
#define TURBOVEC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tv_index tv_index;

/* Status codes.  1..5 are the reference's SearchError variants
 * (turbovec/src/error.rs:234-276). */
typedef enum {
    TV_OK = 0,
    TV_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM = 1, /* lib.rs:1363-1369 */
    TV_ERR_INVALID_QUERY_VALUE = 2,              /* lib.rs:1374-1380, encode.rs:76-83 */
    TV_ERR_MASK_LENGTH_MISMATCH = 3,             /* lib.rs:1427-1434 */
    TV_ERR_ALLOWLIST_EMPTY = 4,                  /* id_map.rs:672 */
    TV_ERR_UNKNOWN_ID = 5,                       /* id_map.rs:677 */
    TV_ERR_BAD_ARGUMENT = 6,                     /* ConstructError / FromPartsError class */
    TV_ERR_HIP = 7,                              /* a HIP runtime call failed */
    TV_ERR_NO_DEVICE = 8,                        /* no gfx950 device visible */
    TV_ERR_INDEX_OUT_OF_RANGE = 9,
    TV_ERR_BAD_IMAGE = 10        /* snapshot bytes refused; tv_last_error says why */
} tv_status;

/* Which integer score definition the scan uses (the reference picks one at run
 * time from CPU features, turbovec/src/pack.rs:1189-1219, search.rs:2975-2980). */
typedef enum {
    TV_SCORE_AUTO = 0,      /* what an AVX-512 VNNI / dotprod host runs: P at 4-bit, L_U32 at 2/3-bit */
    TV_SCORE_L_SCALAR = 1,  /* u8 LUT terms added one by one in f32, bias first   search.rs:3113-3128 (the
                               definition; what FORCE_SCALAR_FALLBACK selects, search.rs:313-316) */
    TV_SCORE_L_CLASSIC = 2, /* u8 LUT sums, fma flush per 256 byte-groups   search.rs:516-582 */
    TV_SCORE_L_U32 = 3,     /* u8 LUT sums, (acc*scale+bias)*vec_scale      search.rs:1174-1177 */
    TV_SCORE_P = 4          /* int8 permute-dot, fma(acc,scale,bias)*vs     search.rs:1519-1524 (4-bit only) */
} tv_score_mode;

const char *tv_status_string(int status);
/* Text of the last HIP failure on the calling thread ("" if none). */
const char *tv_last_error(void);

/* ---- index life cycle -------------------------------------------------- */

/* Replaces the lazily built caches of TurboQuantIndex (lib.rs:1404-1415): the
 * rotation tables (rotation.rs:141-187) and Lloyd-Max centroids
 * (codebook.rs:50) are derived inside and uploaded.  dim: positive multiple of
 * 8, <= 16384; bits in {2,3,4} (lib.rs:629-668).  device: HIP ordinal. */
int tv_index_create(int dim, int bits, int device, tv_index **out);
int tv_index_destroy(tv_index *ix);

/* Hand over the caller's own tables instead of the derived ones: signs and
 * perms are round 0 then round 1 (2*dim each, rotation.rs:110-115), centroids
 * 2^bits values.  Any pointer may be NULL to keep the current table. */
int tv_index_set_tables(tv_index *ix, const float *signs, const uint32_t *perms, const float *centroids);
/* TQ+ pair (lib.rs:329-330), dim values each; both NULL = uncalibrated. */
int tv_index_set_calibration(tv_index *ix, const float *shift, const float *scale);
int tv_index_set_score_mode(tv_index *ix, int mode);

/* Read back the tables in use (for cross-checking against the caller's). */
int tv_index_get_tables(const tv_index *ix, float *signs, uint32_t *perms, float *centroids, float *boundaries);

/* Replace the contents with n_vectors rows given in the sequential-blocked
 * layout the reference persists (pack.rs:336-361: byte of (block b, group g,
 * lane l) at (b*G+g)*32+l, ceil(n/32)*G*32 bytes) and their per-vector scales
 * (lib.rs:312).  Replaces BlockedCache (lib.rs:253-256). */
int tv_index_upload_seq(tv_index *ix, const uint8_t *seq_codes, size_t n_vectors, const float *scales);
/* Same, from device memory (both pointers are device pointers). */
int tv_index_upload_seq_dev(tv_index *ix, const uint8_t *d_seq_codes, size_t n_vectors, const float *d_scales);
/* Append n_new rows; rows[i*G + g] is row i's code byte of group g (the
 * per-vector form extract_codes_flat yields, pack.rs:306).  Replaces
 * append_lanes (pack.rs:211-233). */
int tv_index_append_rows(tv_index *ix, const uint8_t *rows, const float *scales, size_t n_new);
/* Encode n_new raw float rows (n_new*dim values) on the device and append them:
 * normalise, rotate, quantise against the codebook (and the TQ+ pair when one is
 * set), derive the per-vector scale, pack, append.  Codes and scales are
 * bit-identical to the CPU encoder's.  Replaces the encode half of
 * TurboQuantIndex::add (lib.rs:738-966 -> encode.rs:1418-1476, :560-664,
 * :900-932).  Values must be finite with |x| < 1e16 (encode.rs:76-83):
 * TV_ERR_INVALID_QUERY_VALUE otherwise, and nothing is added. */
int tv_index_add(tv_index *ix, const float *vectors, size_t n_new);
/* Fit the TQ+ per-coordinate pair from n >= 2 sample rows and commit it
 * (TurboQuantIndex::calibrate, lib.rs:2599; fit encode.rs:737-857): the sample is
 * normalised and rotated on the device, the order statistics are taken on the
 * host.  Only on an empty index: re-encoding stored rows under a new pair
 * (lib.rs:2599-2835) is not built.  The fitted pair equals the reference's bit
 * for bit. */
int tv_index_calibrate(tv_index *ix, const float *sample, size_t n);
/* The committed pair: *n_calib is 0 (uncalibrated) or dim; shift/scale may be NULL. */
int tv_index_get_calibration(const tv_index *ix, float *shift, float *scale, size_t *n_calib);
/* Same, rows already in device memory (not validated: the caller checked them). */
int tv_index_add_dev(tv_index *ix, const float *d_vectors, size_t n_new);
/* lib.rs:2864-3028: move the last vector into slot idx, zero the vacated lane. */
int tv_index_swap_remove(tv_index *ix, size_t idx);
/* Copy the index back in the sequential-blocked layout (codes_blocked_seq,
 * lib.rs:2088); seq_out holds ceil(n/32)*G*32 bytes, scales_out n floats. */
int tv_index_download_seq(const tv_index *ix, uint8_t *seq_out, float *scales_out);
size_t tv_index_len(const tv_index *ix);
int tv_index_dim(const tv_index *ix);
int tv_index_bits(const tv_index *ix);

/* ---- search ------------------------------------------------------------- */

/* Caller-side validation the reference performs before the seam
 * (lib.rs:1363-1380): len must be a multiple of dim, every value must satisfy
 * |x| < 1e16.  On TV_ERR_INVALID_QUERY_VALUE *bad_index is the flat offset. */
int tv_validate_queries(const float *queries, size_t len, int dim, size_t *bad_index);
/* lib.rs:1435-1456: one byte per slot (non-zero = allowed) to u64 words, LSB =
 * lowest slot; returns the number of allowed slots in *n_allowed. */
int tv_pack_mask(const uint8_t *mask_bytes, size_t n, uint64_t *words_out, size_t *n_allowed);

/* search::search (search.rs:3206).  queries: nq*dim floats.  mask_words: NULL
 * or ceil(n/64) words.  Writes nq*k_eff scores and slot indices, rows sorted
 * (score desc, slot asc), k_eff = min(k, n, popcount(mask)) returned in
 * *out_k_eff; out buffers must hold nq*min(k,n) entries.  k_eff == 0 or
 * nq == 0 writes nothing. */
int tv_search(tv_index *ix, const float *queries, size_t nq, size_t k,
              const uint64_t *mask_words, size_t n_mask_words,
              float *out_scores, int64_t *out_indices, size_t *out_k_eff);

/* Same, with queries, mask words and outputs already in device memory and the
 * mask's popcount supplied by the caller (the reference's caller counts it
 * while packing, lib.rs:1446).  Returns after the work is enqueued and
 * completed on the index's stream. */
int tv_search_dev(tv_index *ix, const float *d_queries, size_t nq, size_t k,
                  const uint64_t *d_mask_words, size_t n_allowed,
                  float *d_out_scores, int64_t *d_out_indices, size_t *out_k_eff);

/* tv_search_dev for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc, code that must not disturb a caching allocator).  No counterpart in the
 * reference.  Like tv_search_dev it runs on the index's own stream and synchronises that stream
 * before it returns (it reads the overflow flags of its passes on the host), so it cannot be
 * recorded into a HIP graph under capture.
 * Same arguments, results and status codes as tv_search_dev, but everything the search carves
 * -- rotated queries, tables, candidate segments, the exact path's lists -- comes out of a
 * fixed array in the library's device image (tv_noalloc_scratch_bytes() bytes, 64 MiB, held by
 * every GPU the library runs on until the process ends), and the call makes no hipMalloc,
 * hipFree, event or stream creation.  A search whose worst case does not fit (at 1536
 * dimensions, 4-bit: more than about 400 queries per call; k > 32 on an index of millions of
 * rows, whose exact fallback ranks dense score rows) is refused with TV_ERR_BAD_ARGUMENT and
 * tv_last_error() names the bytes needed; nothing is written then.  All calls on one GPU share
 * the array: within a process they are serialised by the library; the array keeps the previous
 * call's bytes and every search overwrites what it reads.  Scan timings (tv_last_scan_ms) are
 * not taken on this path. */
int tv_search_dev_noalloc(tv_index *ix, const float *d_queries, size_t nq, size_t k,
                          const uint64_t *d_mask_words, size_t n_allowed,
                          float *d_out_scores, int64_t *d_out_indices, size_t *out_k_eff);
size_t tv_noalloc_scratch_bytes(void);

/* ---- host-only derivations (no GPU touched) ------------------------------- */

/* The tables tv_index_create derives: Rotation::new (rotation.rs:141-187;
 * signs/perms 2*dim each, round 0 first) and codebook::codebook (codebook.rs:50). */
int tv_host_rotation_tables(int dim, float *signs, uint32_t *perms, int *block, float *inv_sqrt_block);
int tv_host_codebook(int bits, int dim, float *boundaries, float *centroids);

/* ---- snapshot images (turbovec/src/io_v7.rs) ------------------------------- */

/* The byte form TurboQuantIndex::to_bytes (lib.rs:2167) / IdMapIndex::to_bytes
 * (id_map.rs:971) and `write` produce: an unclaimed generation-0 TV7 image
 * (io_v7.rs:902-925 write_image: superblock :516-542, header slot :549-599,
 * units :602-629, CRC-32C :128-141).  kind 0 = slot-addressed index, 1 = id map.
 * format 7 is that image; format 6 is the flat TVPI / TVIM container of the
 * release before (convert.rs:14-31, :453-512), which the reference's committed
 * sha256 digests of to_bytes() still hash.  These four touch no GPU. */
size_t tv_host_snapshot_len(int format, int dim, int bits, int kind, size_t n_calib, size_t n);
/* seq: sequential-blocked codes of n rows (what tv_index_download_seq returns);
 * shift/scale: n_calib floats each (n_calib is 0 or dim); ids: n values, kind 1 only.
 * out must hold tv_host_snapshot_len(...) bytes. */
int tv_host_snapshot_compose(int format, int dim, int bits, int kind, const float *boundaries, const float *centroids,
                             size_t n_calib, const float *shift, const float *scale,
                             const uint8_t *seq, size_t n, const float *scales, const uint64_t *ids,
                             uint8_t *out);
/* Validate an image of either format (magic, revision, checksums, geometry, that a TV7
 * image is a snapshot and not a synced container with pending operations) and report its shape. */
int tv_host_snapshot_info(const uint8_t *bytes, size_t len, int *format, int *kind, int *dim, int *bits,
                          size_t *n_calib, size_t *n);
/* Unpack a validated image; any output pointer may be NULL.  seq: ceil(n/32)*G*32 bytes. */
int tv_host_snapshot_extract(const uint8_t *bytes, size_t len, float *boundaries, float *centroids,
                             float *shift, float *scale, uint8_t *seq, float *scales, uint64_t *ids);
/* Snapshot of a device-resident index.  ids == NULL writes kind 0, otherwise kind 1 with
 * ids[slot] (id_map.rs slot_to_id).  out == NULL only reports *len. */
int tv_index_to_bytes(const tv_index *ix, const uint64_t *ids, int format, uint8_t *out, size_t cap, size_t *len);
/* Build a device-resident index from an image (replaces from_v7_image, lib.rs:2196);
 * ids_out (may be NULL) receives n ids for a kind-1 image. */
int tv_index_from_bytes(const uint8_t *bytes, size_t len, int device, tv_index **out, uint64_t *ids_out);

/* ---- test / measurement hooks -------------------------------------------- */

/* Integer accumulators and final float scores of every (query, slot) pair,
 * nq*n each (either may be NULL): what the parity tests compare bit-for-bit. */
int tv_debug_scan(tv_index *ix, const float *queries, size_t nq, int32_t *acc_out, float *scores_out);
/* Query preparation only: rotated (and TQ+-calibrated) rows nq*dim, and per
 * query scale and bias of the active score mode (any may be NULL). */
int tv_debug_prepare(tv_index *ix, const float *queries, size_t nq,
                     float *q_rot_out, float *scale_out, float *bias_out);
/* Duration in milliseconds of the scan kernel launches of the most recent
 * tv_search* call on this index, measured with HIP events on its stream, and
 * how many launches that was. */
int tv_last_scan_ms(const tv_index *ix, float *ms, int *launches);
/* Queries one full-scan launch of the last search served (a full launch of a large batch). */
int tv_debug_queries_per_launch(const tv_index *ix, int *queries);
/* Path selection for tests (results must be identical either way): bit 0 makes
 * every search take the full-range list / dense-select path instead of
 * sample-then-filter; bit 1 keeps large batches on the one-tile-per-launch scan
 * instead of the batched ones; bit 2 keeps them off the all-queries-per-pass
 * kernel only; bit 3 keeps u8-LUT batches on the scan that holds whole tables in
 * LDS (at most 8 queries per pass) instead of the sixteen-query one. */
int tv_debug_set_path(tv_index *ix, int force_full_lists);
/* The sampling ladder a search for the k best of nq queries (its first chunk of up to 1024) runs
 * on this index as it stands, unfiltered: block strides of the successive scans, strides[0 ..
 * *count), the last one 1 (the full scan); level i reads blocks 0, strides[i], 2*strides[i], ...,
 * and in the repeated pass of queries whose candidates overflowed it starts at block
 * repeat_offsets[i].  At most cap entries are written (either array may be NULL); *count = 0 means
 * the search does not sample (large k, or the exact path is forced).  For tests and the bench,
 * which lay rows out against the ladder. */
int tv_debug_sampling_plan(const tv_index *ix, size_t nq, size_t k, uint32_t *strides, uint32_t *repeat_offsets,
                           size_t cap, size_t *count);
/* A sampling level whose candidates do not fit (its floor came from a level that happened to read
 * poor rows) runs a second time, on the device, from the floor taken from what did fit.  track = 1
 * makes searches report such levels (a few hundred bytes more in the flag copy), 0 stops that,
 * negative leaves it as it is; *count (may be NULL) = levels repeated so far while tracking. */
int tv_debug_level_repeats(tv_index *ix, int track, size_t *count);
/* Bytes of the index's cached search workspace and of its host-call staging allocation (either
 * pointer may be NULL): both only ever grow, and tv_search_dev_noalloc touches neither. */
int tv_debug_workspace_bytes(const tv_index *ix, size_t *workspace, size_t *staging);
/* How many queries so far did not finish in the single sampled pass because their
 * candidate buffer overflowed (they are scanned once more, all together, from a raised
 * floor), and how many of those went on to the exact list / select path. */
int tv_debug_overflow_redos(const tv_index *ix, size_t *count);
int tv_debug_exact_redos(const tv_index *ix, size_t *count);
/* How many tv_search / tv_search_dev calls so far were served by another caller's launch: calls
 * that arrive while the index is busy are merged, by the next caller to get it, with every
 * waiting call of the same k and mask into one batch. */
int tv_debug_merged_calls(const tv_index *ix, size_t *count);
/* Bandwidth probe on the index's stream: reps launches of a pure read-sum over
 * d_src (d_dst NULL) or of a plain copy d_src -> d_dst, bytes each; mean
 * milliseconds per launch.  Calibrates the achievable HBM rate and gives the
 * hardware counters a kernel of known traffic. */
int tv_debug_stream_probe(tv_index *ix, const void *d_src, void *d_dst, size_t bytes, int reps, float *ms_per_rep);
/* Matrix-unit probe on the index's stream: reps launches of the batched scan's
 * MFMA loop alone (int8 32x32x32, A operands in registers, B operands read from
 * LDS, pseudo-random bytes, no HBM traffic), iters x 48 MFMAs per wavefront;
 * mean milliseconds per launch and the int8 operations (2 per multiply-add) of
 * one launch.  Calibrates the rate the matrix unit sustains on this chip under
 * its power management, as the read probe does for HBM.  No counterpart in the
 * reference (its roofline probe is the read one, examples/stream_bw.rs:30-66). */
int tv_debug_mfma_probe(tv_index *ix, int iters, int reps, float *ms_per_rep, double *ops_per_rep);
/* Device pointers of the resident index (native layout) for tools. */
int tv_index_device_ptrs(const tv_index *ix, void **d_codes, void **d_scales, size_t *code_bytes);

#ifdef __cplusplus
}
#endif
#endif
