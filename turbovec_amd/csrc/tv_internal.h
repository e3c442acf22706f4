// Internal declarations shared by the HIP kernels and the C-ABI host code.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <condition_variable>
#include <mutex>
#include <vector>

#include "host_tables.h"

namespace tv {

constexpr int kVecBlock = 32;    // vectors per block (turbovec/src/lib.rs:89)
constexpr int kChunkGroups = 32; // byte-groups per native chunk
constexpr int kQTile = 32;       // queries per MFMA column tile
constexpr int kScanThreads = 256;
constexpr int kMaxListK = 32;    // largest k served by the per-lane lists
constexpr int kSegCap = 64;      // candidate keys one workgroup may append per query and launch
constexpr int kFinalCap = 8192;  // candidate keys per query the final sort holds (64 KiB of LDS)
constexpr int kMaxSampledK = 512;   // largest k served by sample-then-filter
constexpr int kTimedLaunches = 32;  // scan launches of one search that are timed with events

// What a scan launch does with the scores it computes.
enum { kModeLists = 0,   // per-lane top-k lists (written out for k_merge)
       kModeDump = 1,    // every score (and accumulator) to dense rows
       kModeAppend = 2,  // every allowed slot scoring >= the query's fixed floor to a candidate buffer
       kModeBest = 3     // per scanned block and query, the best allowed slot to the candidate buffer (no floor)
};

// Native device layout of the codes ("vm32"): the byte of (block b, group g,
// vector i) lives at ((b*nch + g/32)*64 + ((g%32)/16)*32 + i)*16 + g%16, groups
// padded with zero bytes to a multiple of 32.  One 64-lane wave reads a chunk
// (32 vectors x 32 groups = 1 KiB) with one 16-byte load per lane, and the 16
// bytes a lane receives are 16 consecutive groups of ONE vector -- the operand
// shape of the i8 MFMA and of the per-vector LUT walk alike.
struct Geometry {
    int dim = 0, bits = 0;
    int G = 0;    // byte groups per vector = dim*bits/8 (3-bit: dim/2)
    int nch = 0;  // chunks per block: ceil(G/32), plus padding chunks for some 4-bit row lengths (tv_index_create)
    size_t block_bytes() const { return size_t(nch) * 1024; }
};

struct ScanArgs {
    const uint8_t *codes;
    const float *scales;       // padded to a multiple of 32 entries
    const uint64_t *mask;      // nullptr = unfiltered
    const uint8_t *tables;     // this tile's weight fragments (mode P) or LUTs (mode L)
    const float *qscale;       // this tile's per-query scale (kQTile entries)
    const float *qbias;
    int nq_tile;
    uint32_t n;
    uint32_t n_blocks;
    int nch;
    int k;
    uint32_t lv[4];            // the 16 int8 codebook levels, little-endian packed
    int *gtau;                 // kQTile running thresholds (orderable ints)
    float *part_scores;        // [k][total_threads]
    uint32_t *part_idx;
    int *part_cnt;             // [total_threads]
    int32_t *acc_out;          // dump mode: [nq_tile][n] (may be null)
    float *score_out;          // dump mode: [nq_tile][n]
    int classic;               // mode L: 0 = u32 epilogue, 1 = fma flush per 256 groups, 2 = the scalar definition's chain of adds
    int n_groups;              // byte groups of a row that carry codes (the rest of the last chunks is padding)
    uint32_t b_step;           // 1, or a sampling stride: only blocks j*b_step are scanned
    int share_tau;             // lists mode: waves share and raise gtau while scanning
    uint64_t *cand;            // append mode: [nq_tile][seg_stride][kSegCap] sort keys, one segment per workgroup (per four-wave group in the single-tile permute-dot scan)
    uint32_t *cand_cnt;        // append mode: [nq_tile][seg_stride] counts (above kSegCap: that segment overflowed)
    uint32_t seg_stride;       // segments allocated per query (>= grid of the launch)
    uint32_t vgrid;            // single-tile permute-dot scan: four-wave groups of the launch (set by its launcher)
    int best_of_block;         // all-queries-per-pass kernel: no floor, per scanned block and query the best allowed slot (kModeBest)
    const uint32_t *run_if;    // append mode: when given and *run_if == 0 the launch does nothing (a level's conditional repeat)
};

// ---- launchers (tv_kernels.hip) ----
hipError_t launch_seq_to_native(const uint8_t *d_seq, uint8_t *d_native, const Geometry &g, size_t first_block,
                                size_t n_blocks, hipStream_t s);
hipError_t launch_native_to_seq(const uint8_t *d_native, uint8_t *d_seq, const Geometry &g, size_t first_block,
                                size_t n_blocks, hipStream_t s);
hipError_t launch_append_rows(const uint8_t *d_rows, uint8_t *d_native, const Geometry &g, size_t old_n,
                              size_t n_new, hipStream_t s);
hipError_t launch_encode(const float *d_vecs, size_t n_new, size_t old_n, const float *d_signs,
                         const uint32_t *d_perms, const float *d_shift, const float *d_scale,
                         const float *centroids, const float *boundaries, const Geometry &g, int block,
                         float inv_sqrt_block, uint8_t *d_native, float *d_scales, float *d_rot_out,
                         hipStream_t s);
size_t encode_lds_bytes(int dim);
hipError_t launch_move_lane(uint8_t *d_native, float *d_scales, const Geometry &g, size_t src, size_t dst,
                            hipStream_t s);

hipError_t launch_rotate(const float *d_q, float *d_out, const float *d_signs, const uint32_t *d_perms, int dim,
                         int block, float inv_sqrt_block, size_t nq, hipStream_t s);
hipError_t launch_calibrate(const float *d_qrot, float *d_qcal, float *d_bias_corr, const float *d_shift,
                            const float *d_scale, int dim, size_t nq, hipStream_t s);
hipError_t launch_build_p(const float *d_qcal, const float *d_bias_corr, uint8_t *d_wfrag, float *d_qscale,
                          float *d_qbias, int dim, int G, int nch, float cs, size_t nq, size_t nq_padded,
                          bool split, hipStream_t s);
// Rotation, TQ+ inverse (d_shift / d_scale null: none) and permute-dot weights in one launch.
hipError_t launch_prep_p(const float *d_q, const float *d_signs, const uint32_t *d_perms, int dim, int block,
                         float inv_sqrt_block, const float *d_shift, const float *d_scale, uint8_t *d_wfrag,
                         float *d_qscale, float *d_qbias, int G, int nch, float cs, size_t nq, size_t nq_padded, bool split,
                         hipStream_t s);
hipError_t launch_build_lut(const float *d_qcal, const float *d_bias_corr, const float *d_centroids, uint8_t *d_lut,
                            float *d_qscale, float *d_qbias, int dim, int bits, int G, int nch, size_t nq,
                            size_t nq_padded, hipStream_t s);

int scan_grid_blocks(int device, int mode_p, int nch, int k, int lut_queries);
size_t scan_lds_bytes(int mode_p, int nch, int k, int lut_queries);
// Queries one launch of the LUT scan serves (1, 2 or 4), from the LDS budget.
int lut_tile_queries(int nch, int k);
// Queries per LDS entry (1, 2 or 4) the LUT scan launch picks for nq_tile queries.
int lut_launch_ql(int nch, int k, int nq_tile);
int lut_append_queries(int nch);
int lut_append_grid(int device, int nch);
bool lut_single_uses_byte_tables(int nch, int grid);
// Sixteen queries per append-mode pass, score mode L with the u32 or the classic epilogue (tv_kernels4.hip): the
// tables entry-major, 16 bytes per entry, two chunks (32 KiB) after another; chunks padded to even.
constexpr int kLut16Queries = 16;
size_t lut16_table_bytes(int nch, size_t nq);
hipError_t launch_lut_interleave16(const uint8_t *d_src, uint8_t *d_dst, int nch, size_t nq, hipStream_t s);
hipError_t launch_scan_lut16(const ScanArgs &a, int grid, int tiles, hipStream_t s);
int lut16_blocks_per_workgroup(bool classic);   // blocks one workgroup carries through a round of the row's chunks
hipError_t launch_scan_p4(const ScanArgs &a, int grid, int mode, hipStream_t s);
hipError_t launch_scan_lut(const ScanArgs &a, int grid, int mode, hipStream_t s);
// Query tiles one batched permute-dot launch serves for this geometry (0: not available).
int batched_tiles(int nch);
int batched_grid_blocks(int device, int nch);
hipError_t launch_scan_p4_batched(const ScanArgs &a, int grid, hipStream_t s);
bool batched_weights_split(int nch);   // which weight order launch_scan_p4_batched's kernel reads
// out_tau == nullptr: write the k_eff best of the merged lists; else write only the
// order key of the k_eff-th best (a floor at least k_eff scanned slots reach) per query.
// Wide batched scan (every query of a chunk in one pass; tv_kernels3.hip).
int wide_min_queries(int nch);
int wide_grid_blocks(int device);
hipError_t launch_scan_p4_wide(const ScanArgs &a, int grid, hipStream_t s);
int wide_blocks_per_workgroup(int nch);
bool wide_serves_best_of_block(int nch);
int wide_max_queries(int nch);
bool wide_weights_split(int nch);

hipError_t launch_merge(const float *part_scores, const uint32_t *part_idx, const int *part_cnt, int total_threads,
                        int qmod, int k, int k_eff, int nq_tile, float *out_scores, int64_t *out_idx,
                        int *out_tau, hipStream_t s);
// Gathers each query's candidate segments (n_seg of them, seg_stride allocated), sorts, and either
// emits the k_eff best (tau_out == nullptr; a query that did not fit is flagged in overflow) or, for a
// sampling level, writes the order key of the k_floor-th best as the query's next floor to
// tau_out[(q / tau_stride_q) * kQTile + q % tau_stride_q] (keep_floor: a level that gathers fewer than k_eff
// candidates leaves the floor already there in place instead of opening it).  A final pass that
// overflows writes flag 1 and a raised floor to raise_out[q] when raise_out is given (flag 2 and
// nothing otherwise); row_map, when given, names the output row of each query.
// level_over (sampling levels): set to 1 when some query's candidates of this level did not all fit
// (its floor then comes from a subset and may be far too low); clear_flag: a word this launch resets
// to 0 (the flag of the level after); run_if: when given and *run_if == 0 the launch does nothing.
hipError_t launch_final(const uint64_t *cand, const uint32_t *cand_cnt, uint32_t n_seg, uint32_t seg_stride,
                        int k_eff, int k_floor, int nq, float *out_scores, int64_t *out_idx, uint32_t *overflow,
                        int *tau_out, int tau_stride_q, int keep_floor, int *raise_out, const uint32_t *row_map,
                        uint32_t *level_over, uint32_t *clear_flag, const uint32_t *run_if, hipStream_t s);
// Packs the queries rows[0..n_redo) of a chunk and their raised floors for one more full scan.
hipError_t launch_gather_redo(const float *d_q, const uint32_t *d_rows, const int *d_raised, int dim, int tile_q,
                              size_t n_redo, float *d_q_out, int *d_tau_out, hipStream_t s);
hipError_t launch_fill_i32(int *p, int v, size_t n, hipStream_t s);
hipError_t launch_probe(const void *src, void *dst, size_t bytes, int copy, uint32_t *sink, hipStream_t s);
hipError_t launch_probe_mfma(int device, int iters, uint32_t *sink, double *ops, hipStream_t s);
// Exact top-k of a dense score row per query (NaN = excluded slot).
hipError_t launch_select_topk(const float *d_scores, size_t n, int nq_tile, size_t k_eff, uint64_t *d_keys_tmp,
                              uint32_t *d_hist, float *out_scores, int64_t *out_idx, hipStream_t s);
size_t select_tmp_keys(size_t k_eff);

}  // namespace tv

struct tv_request;   // a search call waiting for the index (tv_api.hip)

// The opaque handle of the C ABI.
struct tv_index {
    tv::Geometry geo;
    int device = 0;
    int score_mode = 0;
    tv::RotationTables rot;
    tv::Codebook cb;
    std::vector<float> tq_shift, tq_scale;
    int8_t levels[16] = {0};
    float cs = 1.0f;

    hipStream_t stream = nullptr;
    hipEvent_t ev_start[tv::kTimedLaunches] = {}, ev_stop[tv::kTimedLaunches] = {};
    bool events_ready = false;
    float *d_signs = nullptr;
    uint32_t *d_perms = nullptr;
    float *d_centroids = nullptr;
    float *d_tq_shift = nullptr, *d_tq_scale = nullptr;
    int *d_tau_open = nullptr;     // order key of -inf per query: the floors before any level has run

    uint8_t *d_codes = nullptr;
    float *d_scales = nullptr;
    size_t cap_blocks = 0;
    size_t n = 0;

    // Search calls that arrived while another held the index: whoever takes `mu` next serves every
    // waiting call that asks for the same k under the same mask together with its own, as one batch.
    std::mutex waiting_mu;
    std::condition_variable waiting_cv;   // a call registered, or a batch was served
    std::vector<tv_request *> waiting;
    bool serving = false;          // some caller is serving a batch right now
    size_t last_batch_calls = 0;   // calls in the batch served last: how many callers to expect again shortly
    size_t merged_calls = 0;       // calls that were served by another caller's launch

    // per-search workspace, grown on demand, guarded by mu
    mutable std::mutex mu;
    void *ws = nullptr;
    void *io = nullptr;            // staging for tv_search's host buffers (queries, mask, results); grows, never shrinks
    size_t io_bytes = 0;
    size_t ws_bytes = 0;
    bool ws_fixed = false;         // ws is a lent buffer of fixed size (tv_search_dev_noalloc): never reallocated
    void *scratch = nullptr;       // this device's copy of the library's static scratch array
    uint32_t *h_flags = nullptr;   // pinned host memory: the overflow flags of one group of chunks, then the rows to repeat
    uint32_t *d_flags_host = nullptr;   // the device's address of h_flags
    size_t exact_redos = 0;        // queries that went on to the exact path
    float last_scan_ms = 0.0f;
    int last_scan_launches = 0;
    int last_queries_per_launch = 0;   // queries one full-scan launch of the last search served
    int force_robust = 0;          // test hook: skip sample-then-filter
    int no_batched = 0;            // test hook: one query tile per scan launch even for large batches
    int no_lut16 = 0;              // test hook: mode L batches stay on the scan with whole tables in LDS (8 queries per pass at most)
    int no_wide = 0;               // test hook: large batches go through the tile-group kernels, not the wide one
    size_t overflow_redos = 0;     // queries redone because their candidate buffer overflowed
    // The floorless first level (best row per block) misjudges the floor when a query's neighbours
    // sit together in a few blocks (a clustered corpus in insertion order): after a search in which
    // it made an eighth of the queries overflow, the next searches run the ladder of row-level
    // samples instead, and the floorless level gets another try afterwards.  When the row-level
    // ladder then fails the same way (rows laid out against its strides), the floorless level comes
    // back at once and stays for as many searches: its failure costs less.
    int row_ladder_left = 0;
    int floorless_kept_left = 0;
    int track_levels = 0;          // test hook: read the per-level flags back with the overflow flags and count them
    size_t level_repeats = 0;      // sampling levels that ran a second time because their candidates did not fit
};
