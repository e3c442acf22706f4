// C ABI of the search path (see include/turbovec_hip.h).
#include "../../include/turbovec_hip.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <new>
#include <string>
#include <vector>

#include "tv_internal.h"
#include "tv_snapshot.h"

namespace {

thread_local std::string g_last_error;

int fail_hip(hipError_t e, const char *what) {
    char buf[256];
    snprintf(buf, sizeof buf, "%s: %s", what, hipGetErrorString(e));
    g_last_error = buf;
    return TV_ERR_HIP;
}

#define TV_HIP(call)                                        \
    do {                                                    \
        hipError_t e__ = (call);                            \
        if (e__ != hipSuccess) return fail_hip(e__, #call); \
    } while (0)

size_t round_up(size_t v, size_t m) { return (v + m - 1) / m * m; }

// Bump allocator over the index's cached workspace.
struct Arena {
    uint8_t *base = nullptr;
    size_t used = 0;
    template <typename T>
    T *take(size_t count) {
        T *p = reinterpret_cast<T *>(base + used);
        used += round_up(count * sizeof(T), 256);
        return p;
    }
};

// ---- the scratch buffer of tv_search_dev_noalloc ---------------------------------------------
// One array per GPU, in the library's device image: every device the library runs on holds
// kScratchBytes of it from the moment the image is loaded there until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress; each device's copy has an
// address of its own, looked up once per device and kept in g_scratch.
constexpr size_t kScratchBytes = size_t(64) << 20;
static __device__ __align__(256) uint8_t scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
struct DeviceScratch {
    void *ptr = nullptr;     // device address of `scratch` on this device
    std::mutex in_use;       // calls on one device share the array: one at a time within the process
};
DeviceScratch g_scratch[kMaxDevices];
std::mutex g_scratch_setup;

// Device `device` must be current.
int scratch_address(int device, void **out) {
    if (device < 0 || device >= kMaxDevices) { g_last_error = "device ordinal beyond the scratch table"; return TV_ERR_NO_DEVICE; }
    std::lock_guard<std::mutex> lock(g_scratch_setup);
    if (!g_scratch[device].ptr) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return fail_hip(e, "hipGetSymbolAddress(scratch)");
        g_scratch[device].ptr = p;
    }
    *out = g_scratch[device].ptr;
    return TV_OK;
}

int ensure_workspace(tv_index *ix, size_t bytes) {
    if (bytes <= ix->ws_bytes) return TV_OK;
    if (ix->ws_fixed) {   // the caller lent a buffer of fixed size: never replaced
        g_last_error = "search needs " + std::to_string(bytes) + " bytes of scratch, the fixed buffer holds " +
                       std::to_string(ix->ws_bytes);
        return TV_ERR_BAD_ARGUMENT;
    }
    if (ix->ws) { TV_HIP(hipFree(ix->ws)); ix->ws = nullptr; ix->ws_bytes = 0; }
    bytes = round_up(bytes + bytes / 4, size_t(1) << 20);
    TV_HIP(hipMalloc(&ix->ws, bytes));
    ix->ws_bytes = bytes;
    return TV_OK;
}

int ensure_io(tv_index *ix, size_t bytes) {
    if (bytes <= ix->io_bytes) return TV_OK;
    if (ix->io) { TV_HIP(hipFree(ix->io)); ix->io = nullptr; ix->io_bytes = 0; }
    bytes = round_up(bytes + bytes / 4, size_t(1) << 16);
    TV_HIP(hipMalloc(&ix->io, bytes));
    ix->io_bytes = bytes;
    return TV_OK;
}

int ensure_capacity(tv_index *ix, size_t n_vectors) {
    const size_t blocks = (n_vectors + tv::kVecBlock - 1) / tv::kVecBlock;
    if (blocks <= ix->cap_blocks) return TV_OK;
    size_t cap = std::max(blocks, ix->cap_blocks + ix->cap_blocks / 2);
    cap = std::max<size_t>(cap, 64);
    uint8_t *codes = nullptr;
    float *scales = nullptr;
    const size_t bb = ix->geo.block_bytes();
    TV_HIP(hipMalloc(reinterpret_cast<void **>(&codes), cap * bb));
    {
        const hipError_t e = hipMalloc(reinterpret_cast<void **>(&scales), cap * tv::kVecBlock * sizeof(float));
        if (e != hipSuccess) {
            (void)hipFree(codes);
            return fail_hip(e, "hipMalloc(scales)");
        }
    }
    const size_t old_blocks = (ix->n + tv::kVecBlock - 1) / tv::kVecBlock;
    // fresh bytes are zero so padding lanes match a from-scratch upload
    TV_HIP(hipMemsetAsync(codes + old_blocks * bb, 0, (cap - old_blocks) * bb, ix->stream));
    TV_HIP(hipMemsetAsync(scales + old_blocks * tv::kVecBlock, 0,
                          (cap - old_blocks) * tv::kVecBlock * sizeof(float), ix->stream));
    if (old_blocks) {
        TV_HIP(hipMemcpyAsync(codes, ix->d_codes, old_blocks * bb, hipMemcpyDeviceToDevice, ix->stream));
        TV_HIP(hipMemcpyAsync(scales, ix->d_scales, old_blocks * tv::kVecBlock * sizeof(float),
                              hipMemcpyDeviceToDevice, ix->stream));
    }
    TV_HIP(hipStreamSynchronize(ix->stream));
    if (ix->d_codes) TV_HIP(hipFree(ix->d_codes));
    if (ix->d_scales) TV_HIP(hipFree(ix->d_scales));
    ix->d_codes = codes;
    ix->d_scales = scales;
    ix->cap_blocks = cap;
    return TV_OK;
}

// An upload replaces the contents: blocks of the old contents beyond the new end are cleared, so
// that rows appended later land in zeroed blocks (padding lanes zero, as in a from-scratch
// upload; pack.rs:235-243, :354).
int clear_tail_blocks(tv_index *ix, size_t n_blocks) {
    if (n_blocks >= ix->cap_blocks) return TV_OK;
    const size_t bb = ix->geo.block_bytes();
    TV_HIP(hipMemsetAsync(ix->d_codes + n_blocks * bb, 0, (ix->cap_blocks - n_blocks) * bb, ix->stream));
    TV_HIP(hipMemsetAsync(ix->d_scales + n_blocks * tv::kVecBlock, 0,
                          (ix->cap_blocks - n_blocks) * tv::kVecBlock * sizeof(float), ix->stream));
    return TV_OK;
}

// turbovec/src/search.rs:2812-2820: the codebook as int8 levels, one scale.
void derive_levels(tv_index *ix) {
    float cmax = 0.0f;
    for (float c : ix->cb.centroids) cmax = std::fmax(cmax, std::fabs(c));
    ix->cs = cmax > 0.0f ? cmax / 127.0f : 1.0f;
    std::memset(ix->levels, 0, sizeof ix->levels);
    for (size_t i = 0; i < ix->cb.centroids.size() && i < 16; ++i) {
        float v = std::round(ix->cb.centroids[i] / ix->cs);
        v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
        ix->levels[i] = int8_t(v);
    }
}

int upload_tables(tv_index *ix) {
    const size_t dim = size_t(ix->geo.dim);
    TV_HIP(hipMemcpyAsync(ix->d_signs, ix->rot.signs.data(), 2 * dim * sizeof(float), hipMemcpyHostToDevice,
                          ix->stream));
    TV_HIP(hipMemcpyAsync(ix->d_perms, ix->rot.perms.data(), 2 * dim * sizeof(uint32_t), hipMemcpyHostToDevice,
                          ix->stream));
    float cen[16] = {0};
    for (size_t i = 0; i < ix->cb.centroids.size(); ++i) cen[i] = ix->cb.centroids[i];
    TV_HIP(hipMemcpyAsync(ix->d_centroids, cen, sizeof cen, hipMemcpyHostToDevice, ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    return TV_OK;
}

int effective_mode(const tv_index *ix);
// Queries one LUT-scan launch serves: the scalar definition's float chain runs one query at a time.
int lut_tile_q(const tv_index *ix, int k) { return effective_mode(ix) == TV_SCORE_L_SCALAR ? 1 : tv::lut_tile_queries(ix->geo.nch, k); }
// Queries one append-mode LUT launch serves: sixteen with the u32 and the classic epilogues (tables
// streamed through LDS), one for the scalar definition's chain.
bool lut16_serves(const tv_index *ix) {
    return (effective_mode(ix) == TV_SCORE_L_U32 || effective_mode(ix) == TV_SCORE_L_CLASSIC) && !ix->no_lut16;
}
int lut_append_q(const tv_index *ix) {
    if (effective_mode(ix) == TV_SCORE_L_SCALAR) return 1;
    return lut16_serves(ix) ? tv::kLut16Queries : tv::lut_append_queries(ix->geo.nch);
}
// Tiles of fewer queries than this keep the whole-table scan (its pass is as long for 8 queries as for 1).
constexpr int kLut16MinQueries = 9;

int effective_mode(const tv_index *ix) {
    int m = ix->score_mode;
    if (m == TV_SCORE_AUTO) m = ix->geo.bits == 4 ? TV_SCORE_P : TV_SCORE_L_U32;
    return m;
}

struct Prepared {
    float *d_qrot = nullptr;   // rotated (and calibrated) rows
    uint8_t *d_tables = nullptr;
    uint8_t *d_tables16 = nullptr;   // mode L: the same tables entry-major for the sixteen-query scan (or null)
    float *d_qscale = nullptr, *d_qbias = nullptr;
    size_t table_bytes_per_tile = 0;
};

// Query preparation for one chunk: rotation, TQ+ inverse, table build
// (turbovec/src/search.rs:3237-3269).  d_q holds nq*dim floats on the device.
// `split`: permute-dot weights in the order k_scan_p4 reads them (the batched scans take plane order)
// `keep_rotated`: the rotated rows are wanted in device memory too (the debug read-back); a search
// in permute-dot mode does not need them and prepares its queries in a single launch.
// `for_append`: u8-LUT tables are wanted entry-major too, for the sixteen-query append scan.
int prepare_queries(tv_index *ix, Arena &ar, const float *d_q, size_t nq, Prepared &out, bool split = true,
                    bool keep_rotated = false, bool for_append = false) {
    const tv::Geometry &g = ix->geo;
    const size_t nq_pad = round_up(nq, tv::kQTile);
    const int mode = effective_mode(ix);
    if (mode == TV_SCORE_P && !keep_rotated) {
        const bool cal = !ix->tq_shift.empty();
        out.d_qrot = nullptr;
        out.d_qscale = ar.take<float>(nq_pad);
        out.d_qbias = ar.take<float>(nq_pad);
        out.table_bytes_per_tile = size_t(g.nch) * 2048;
        out.d_tables = ar.take<uint8_t>(nq_pad / tv::kQTile * out.table_bytes_per_tile);
        TV_HIP(tv::launch_prep_p(d_q, ix->d_signs, ix->d_perms, g.dim, ix->rot.block, ix->rot.inv_sqrt_block,
                                 cal ? ix->d_tq_shift : nullptr, cal ? ix->d_tq_scale : nullptr, out.d_tables, out.d_qscale,
                                 out.d_qbias, g.G, g.nch, ix->cs, nq, nq_pad, split, ix->stream));
        return TV_OK;
    }
    float *d_rot = ar.take<float>(nq * g.dim);
    float *d_bias_corr = ar.take<float>(nq_pad);
    TV_HIP(tv::launch_rotate(d_q, d_rot, ix->d_signs, ix->d_perms, g.dim, ix->rot.block, ix->rot.inv_sqrt_block, nq,
                             ix->stream));
    float *d_cal = d_rot;
    if (!ix->tq_shift.empty()) {
        d_cal = ar.take<float>(nq * g.dim);
        TV_HIP(tv::launch_calibrate(d_rot, d_cal, d_bias_corr, ix->d_tq_shift, ix->d_tq_scale, g.dim, nq,
                                    ix->stream));
    } else {
        d_bias_corr = nullptr;   // uncalibrated: the table builders add +0.0f themselves (search.rs:3176-3185)
    }
    out.d_qrot = d_cal;
    out.d_qscale = ar.take<float>(nq_pad);
    out.d_qbias = ar.take<float>(nq_pad);
    if (mode == TV_SCORE_P) {
        out.table_bytes_per_tile = size_t(g.nch) * 2048;
        out.d_tables = ar.take<uint8_t>(nq_pad / tv::kQTile * out.table_bytes_per_tile);
        TV_HIP(tv::launch_build_p(d_cal, d_bias_corr, out.d_tables, out.d_qscale, out.d_qbias, g.dim, g.G, g.nch,
                                  ix->cs, nq, nq_pad, split, ix->stream));
    } else {
        out.table_bytes_per_tile = size_t(g.nch) * 1024 * tv::kQTile;
        out.d_tables = ar.take<uint8_t>(nq_pad * size_t(g.nch) * 1024);
        TV_HIP(tv::launch_build_lut(d_cal, d_bias_corr, ix->d_centroids, out.d_tables, out.d_qscale, out.d_qbias,
                                    g.dim, g.bits, g.G, g.nch, nq, nq_pad, ix->stream));
        if (for_append && lut16_serves(ix) && nq >= size_t(kLut16MinQueries)) {
            out.d_tables16 = ar.take<uint8_t>(tv::lut16_table_bytes(g.nch, nq));
            TV_HIP(tv::launch_lut_interleave16(out.d_tables, out.d_tables16, g.nch, nq, ix->stream));
        }
    }
    return TV_OK;
}

size_t prepare_bytes(const tv_index *ix, size_t nq) {
    const tv::Geometry &g = ix->geo;
    const size_t nq_pad = round_up(nq, tv::kQTile);
    size_t b = 2 * round_up(nq * g.dim * 4, 256) + 3 * round_up(nq_pad * 4, 256);
    b += round_up(nq_pad * size_t(g.nch) * 1024, 256) + 4096;
    if (lut16_serves(ix)) b += round_up(tv::lut16_table_bytes(g.nch, nq), 256);
    return b;
}

void fill_scan_args(const tv_index *ix, tv::ScanArgs &a) {
    std::memset(&a, 0, sizeof a);
    a.codes = ix->d_codes;
    a.scales = ix->d_scales;
    a.n = uint32_t(ix->n);
    a.n_blocks = uint32_t((ix->n + tv::kVecBlock - 1) / tv::kVecBlock);
    a.nch = ix->geo.nch;
    std::memcpy(a.lv, ix->levels, 16);
    a.classic = effective_mode(ix) == TV_SCORE_L_CLASSIC ? 1 : effective_mode(ix) == TV_SCORE_L_SCALAR ? 2 : 0;
    a.n_groups = ix->geo.G;
    a.b_step = 1;
}

constexpr size_t kChunkQueries = 1024;
// a chunk's floors are laid out tile by tile, kQTile slots per tile, and a tile may hold one query
constexpr size_t kTauOpenInts = kChunkQueries * tv::kQTile;
constexpr int kMaxTimedTiles = int(kChunkQueries / tv::kQTile);

static_assert(kMaxTimedTiles == tv::kTimedLaunches, "the index holds one event pair per timed launch");

// The events that time scan launches belong to the index (created on first use under its lock,
// destroyed with it).
int ensure_events(tv_index *ix) {
    if (ix->events_ready) return TV_OK;
    for (int i = 0; i < kMaxTimedTiles; ++i) {
        TV_HIP(hipEventCreate(&ix->ev_start[i]));
        TV_HIP(hipEventCreate(&ix->ev_stop[i]));
    }
    ix->events_ready = true;
    return TV_OK;
}

// Workspace bytes one chunk of cq queries needs on the exact path (search_robust) ...
size_t robust_need(const tv_index *ix, size_t cq, size_t k_eff) {
    const tv::Geometry &g = ix->geo;
    const bool mode_p = effective_mode(ix) == TV_SCORE_P;
    const bool lists = k_eff <= size_t(tv::kMaxListK);
    const int kl = lists ? int(k_eff) : 1;
    const size_t tile_q = mode_p ? size_t(tv::kQTile) : size_t(lut_tile_q(ix, kl));
    const size_t n_tiles = (cq + tile_q - 1) / tile_q;
    const int grid = tv::scan_grid_blocks(ix->device, mode_p, g.nch, kl, int(tile_q));
    const size_t total_threads = size_t(grid) * tv::kScanThreads;
    size_t need = prepare_bytes(ix, cq) + round_up(n_tiles * tv::kQTile * 4, 256);
    if (lists) need += 2 * round_up(k_eff * total_threads * 4, 256) + round_up(total_threads * 4, 256);
    else need += round_up(size_t(tv::kQTile) * ix->n * 4, 256) + round_up(tv::select_tmp_keys(k_eff) * 8 * tv::kQTile, 256) +
                 round_up(size_t(tv::kQTile) * 4096 * 4, 256);
    return need + 65536;
}

// ... and on the sampled path (search_device): prepared queries, floors, candidate segments.
struct SampledPlan {
    size_t tile_q, n_tiles, cq_pad, seg_stride, need;
    bool wide;
    bool lut16;         // u8-LUT tiles of this chunk take the sixteen-query scan
    bool lut_single;    // one u8-LUT query, served by the byte-table scan
    int nt_batched;     // query tiles one launch of the tile-group kernels serves (0: one tile per launch)
    int grid;
};
SampledPlan sampled_plan(const tv_index *ix, size_t cq) {
    const tv::Geometry &g = ix->geo;
    const bool mode_p = effective_mode(ix) == TV_SCORE_P;
    SampledPlan p;
    p.tile_q = mode_p ? size_t(tv::kQTile) : size_t(lut_append_q(ix));
    p.n_tiles = (cq + p.tile_q - 1) / p.tile_q;
    p.cq_pad = p.n_tiles * p.tile_q;
    // large chunks of high-dimensional queries take the wide kernel: all of them in one pass per level
    const int wide_min = tv::wide_min_queries(g.nch);
    p.wide = mode_p && !ix->no_batched && !ix->no_wide && wide_min > 0 && cq >= size_t(wide_min);
    p.lut16 = !mode_p && lut16_serves(ix) && cq >= size_t(kLut16MinQueries);
    p.nt_batched = (mode_p && cq > size_t(tv::kQTile) && !ix->no_batched) ? tv::batched_tiles(g.nch) : 0;
    p.grid = p.wide ? tv::wide_grid_blocks(ix->device)
           : mode_p ? tv::scan_grid_blocks(ix->device, mode_p, g.nch, 0, int(p.tile_q))
                    : tv::lut_append_grid(ix->device, g.nch);
    p.lut_single = !mode_p && cq == 1 && effective_mode(ix) != TV_SCORE_L_SCALAR && tv::lut_single_uses_byte_tables(g.nch, p.grid);
    p.seg_stride = size_t(p.grid);
    // (a query keeps one candidate segment per workgroup of the launches that serve it: every launch
    // of a chunk the tile-group kernels serve is one of theirs, and their grid is not the single-tile scan's)
    if (p.nt_batched > 0 && !p.wide) p.seg_stride = size_t(tv::batched_grid_blocks(ix->device, g.nch));
    p.need = prepare_bytes(ix, cq) + round_up(p.n_tiles * tv::kQTile * 4, 256) +
             round_up(p.cq_pad * p.seg_stride * tv::kSegCap * 8, 256) + round_up(p.cq_pad * p.seg_stride * 4, 256) +
             round_up(p.cq_pad * 4, 256) + 65536;
    return p;
}

// Sampling plan of a search: block strides of the successive append-mode scans,
// the last one being 1 (the full scan).  The first level reads about `first`
// slots and, having no floor yet, appends all of them (one short sort); level
// sizes then grow geometrically to the full index, by a factor chosen so that
// a level filtered by the floor of the one before appends at most about 4096
// candidates per query (the floor is the k_floor-th best of the level before,
// so a level `ratio` times larger keeps about ratio * k_floor).  The sampling
// levels together read about 1/ratio of the index.
struct SamplingSteps {
    static constexpr int kMax = 32;   // levels grow at least fourfold: 2^31 slots need 16 at most
    uint32_t step[kMax];
    size_t count = 0;
    bool best_first = false;   // the first level runs without floors and hands over the best row of every block it reads
    size_t size() const { return count; }
    uint32_t operator[](size_t i) const { return step[i]; }
};
// `round_blocks` > 0: the scan kernel works through the blocks in rounds of that many (one per
// wave of the grid) and a level costs whole rounds whatever it fills of the last one; a level
// larger than a round is trimmed to whole rounds (its floor gets a little lower, the next level
// a little longer: at 10M rows 3157 blocks become 2048, one round instead of two).
SamplingSteps sampling_steps(size_t n_blocks, size_t k_floor, size_t round_blocks = 0) {
    const double n_slots = double(n_blocks * tv::kVecBlock);
    const double first = double(std::max<size_t>(1024, 8 * k_floor));
    SamplingSteps steps;
    if (n_slots > 2.0 * first) {
        const double max_ratio = std::max(4.0, double(tv::kFinalCap / 2) / double(k_floor));
        const int levels = std::max(1, int(std::ceil(std::log(n_slots / first) / std::log(max_ratio))));
        const double ratio = std::pow(n_slots / first, 1.0 / double(levels));
        double sample = first;
        for (int lv = 0; lv < levels && steps.count + 1 < size_t(SamplingSteps::kMax); ++lv, sample *= ratio) {
            size_t sample_blocks = std::max<size_t>(1, size_t(sample) / tv::kVecBlock);
            if (round_blocks > 0 && sample_blocks > round_blocks) sample_blocks -= sample_blocks % round_blocks;
            // a trimmed level must not spill into one more round: step rounded up
            const size_t step = round_blocks > 0 && sample_blocks >= round_blocks ? (n_blocks + sample_blocks - 1) / sample_blocks
                                                                                  : n_blocks / sample_blocks;
            if (step > 1 && (steps.count == 0 || step < steps.step[steps.count - 1])) steps.step[steps.count++] = uint32_t(step);
        }
    }
    steps.step[steps.count++] = 1;
    return steps;
}

// The all-queries-per-pass kernel holds 16 bytes of LDS per query beside its slice ring: a call with
// more than kChunkQueries queries left takes them up to kWideChunkQueries at a time there -- a block
// is then loaded and decoded once per 64 query tiles instead of once per 32.
constexpr size_t kWideChunkQueries = 2 * kChunkQueries;      // (where the instance for the row length fits that many)
bool wide_serves(const tv_index *ix) {
    return effective_mode(ix) == TV_SCORE_P && !ix->no_batched && !ix->no_wide && tv::wide_min_queries(ix->geo.nch) > 0;
}
size_t chunk_len(const tv_index *ix, size_t remaining) {
    if (remaining > kChunkQueries && wide_serves(ix))
        return std::min(remaining, std::min<size_t>(kWideChunkQueries, size_t(tv::wide_max_queries(ix->geo.nch))));
    return std::min(remaining, kChunkQueries);
}

// Queries of one call are processed in chunks (chunk_len); the chunks of a group are enqueued
// back to back and the host reads their overflow flags once, after the group's last chunk.
constexpr size_t kGroupQueries = 8 * kChunkQueries;
constexpr size_t kLevelFlagWords = (kGroupQueries / kChunkQueries) * SamplingSteps::kMax;   // per chunk, one word per level

// What a group keeps at the head of the workspace across its passes: per query the overflow flag and
// the raised floor of the first pass; for the repeated pass the rows to repeat and their queries
// packed (one chunk's worth at a time); the per-level "candidates did not fit" flags of the pass in
// flight.
size_t group_header_bytes(const tv_index *ix, size_t gq) {
    const size_t cq = std::min(gq, kWideChunkQueries);
    return 2 * round_up(gq * 4, 256) + round_up(cq * 4, 256) + round_up(cq * size_t(ix->geo.dim) * 4, 256) +
           round_up(kLevelFlagWords * 4, 256);
}

// Workspace the sampled path needs for a call of nq queries: the header of its largest group, the
// working set of a full chunk (or of the only, smaller one), and room for the repeated pass to run
// at least a tile of queries at a time (a smaller packed batch may fall to another kernel with
// more candidate segments per query; it is then cut into pieces that fit).
constexpr size_t kRepeatPieces[] = {1024, 512, 256, 128, 96, 64, 32};
size_t sampled_need_worst(const tv_index *ix, size_t nq) {
    const size_t gq = std::min(nq, kGroupQueries);
    size_t need = 0;
    auto chunks_of_group = [&](size_t group_queries) {
        for (size_t c0 = 0; c0 < group_queries;) {
            const size_t cq = chunk_len(ix, group_queries - c0);
            need = std::max(need, sampled_plan(ix, cq).need);
            c0 += cq;
        }
    };
    chunks_of_group(gq);                                                              // a full group, or the only one
    if (nq > kGroupQueries && nq % kGroupQueries != 0) chunks_of_group(nq % kGroupQueries);   // and the last, shorter one
    need = std::max(need, sampled_plan(ix, std::min<size_t>(nq, tv::kQTile)).need);
    return need + group_header_bytes(ix, gq);
}

// Full-range search without sampling: per-lane lists with shared thresholds for
// k <= 32, dense scores + radix select beyond.  Always exact; used for the
// queries whose candidate buffer overflowed and for very large k.
int search_robust(tv_index *ix, const float *d_queries, size_t nq, size_t k_eff, const uint64_t *d_mask,
                  float *d_out_scores, int64_t *d_out_idx, bool timed_run) {
    const size_t n = ix->n;
    const tv::Geometry &g = ix->geo;
    const int mode = effective_mode(ix);
    const bool mode_p = mode == TV_SCORE_P;
    const bool lists = k_eff <= size_t(tv::kMaxListK);
    int rc = TV_OK;
    for (size_t q0 = 0; q0 < nq; q0 += kChunkQueries) {
        const size_t cq = std::min(kChunkQueries, nq - q0);
        const int kl = lists ? int(k_eff) : 1;
        const size_t tile_q = mode_p ? size_t(tv::kQTile) : size_t(lut_tile_q(ix, kl));
        const size_t n_tiles = (cq + tile_q - 1) / tile_q;
        const int grid = tv::scan_grid_blocks(ix->device, mode_p, g.nch, kl, int(tile_q));
        const size_t total_threads = size_t(grid) * tv::kScanThreads;
        rc = ensure_workspace(ix, robust_need(ix, cq, k_eff));
        if (rc != TV_OK) return rc;
        Arena ar;
        ar.base = static_cast<uint8_t *>(ix->ws);
        Prepared pq;
        rc = prepare_queries(ix, ar, d_queries + q0 * g.dim, cq, pq);
        if (rc != TV_OK) return rc;
        int *d_tau = ar.take<int>(n_tiles * tv::kQTile);
        TV_HIP(tv::launch_fill_i32(d_tau, int(0x807fffffu) /* order key of -inf */, n_tiles * tv::kQTile, ix->stream));
        float *d_part_s = nullptr, *d_dense = nullptr;
        uint32_t *d_part_i = nullptr, *d_hist = nullptr;
        int *d_part_c = nullptr;
        uint64_t *d_keys = nullptr;
        if (lists) {
            d_part_s = ar.take<float>(k_eff * total_threads);
            d_part_i = ar.take<uint32_t>(k_eff * total_threads);
            d_part_c = ar.take<int>(total_threads);
        } else {
            d_dense = ar.take<float>(size_t(tv::kQTile) * n);
            d_keys = ar.take<uint64_t>(tv::select_tmp_keys(k_eff) * tv::kQTile);
            d_hist = ar.take<uint32_t>(size_t(tv::kQTile) * 4096);
        }
        for (size_t t = 0; t < n_tiles; ++t) {
            tv::ScanArgs a;
            fill_scan_args(ix, a);
            a.mask = d_mask;
            a.tables = pq.d_tables + t * (mode_p ? pq.table_bytes_per_tile : tile_q * size_t(g.nch) * 1024);
            a.qscale = pq.d_qscale + t * tile_q;
            a.qbias = pq.d_qbias + t * tile_q;
            a.nq_tile = int(std::min<size_t>(tile_q, cq - t * tile_q));
            a.k = kl;
            a.gtau = d_tau + t * tv::kQTile;
            a.part_scores = d_part_s; a.part_idx = d_part_i; a.part_cnt = d_part_c;
            a.score_out = d_dense;
            a.share_tau = 1;
            if (!lists && d_mask)  // blocks without an allowed slot are skipped by the scan: mark them excluded
                TV_HIP(tv::launch_fill_i32(reinterpret_cast<int *>(d_dense), 0x7fc00000, size_t(a.nq_tile) * n, ix->stream));
            const bool timed = timed_run && int(t) < kMaxTimedTiles;
            const int smode = lists ? tv::kModeLists : tv::kModeDump;
            if (timed) TV_HIP(hipEventRecord(ix->ev_start[t], ix->stream));
            if (mode_p) TV_HIP(tv::launch_scan_p4(a, grid, smode, ix->stream));
            else TV_HIP(tv::launch_scan_lut(a, grid, smode, ix->stream));
            if (timed) TV_HIP(hipEventRecord(ix->ev_stop[t], ix->stream));
            float *os = d_out_scores + (q0 + t * tile_q) * k_eff;
            int64_t *oi = d_out_idx + (q0 + t * tile_q) * k_eff;
            if (lists) {
                const int qmod = mode_p ? tv::kQTile : mode == TV_SCORE_L_SCALAR ? 1 : tv::lut_launch_ql(g.nch, kl, a.nq_tile);
                TV_HIP(tv::launch_merge(d_part_s, d_part_i, d_part_c, int(total_threads), qmod, int(k_eff), int(k_eff),
                                        a.nq_tile, os, oi, nullptr, ix->stream));
            } else {
                TV_HIP(tv::launch_select_topk(d_dense, n, a.nq_tile, k_eff, d_keys, d_hist, os, oi, ix->stream));
            }
        }
        TV_HIP(hipStreamSynchronize(ix->stream));
        for (size_t t = 0; timed_run && t < n_tiles && int(t) < kMaxTimedTiles; ++t) {
            float ms = 0.0f;
            TV_HIP(hipEventElapsedTime(&ms, ix->ev_start[t], ix->ev_stop[t]));
            ix->last_scan_ms += ms;
            ix->last_scan_launches += 1;
        }
    }
    return TV_OK;
}

// Block strides of the sampling ladder a first pass over cq queries runs (the last one is 1).  The
// all-queries-per-pass kernel works through the blocks in rounds of its grid, and its levels are
// trimmed to whole rounds.
//
// A first pass served by the single-tile permute-dot kernel (up to 32 queries), the all-queries
// kernel or the single-query byte-table LUT scan runs one sampling level only, without a floor:
// the scan hands over the best row of every block it reads (kModeBest), and the k_floor-th best
// of those is the floor of the full scan.  The level is sized so that the full scan then appends
// about 2048 rows per query (1024 on the all-queries kernel), and reads at least 8 * k_floor
// blocks; a quarter of the index or more is not worth sampling.
constexpr size_t kBestLevelMaxK = 64;
constexpr size_t kBestLevelMaxKLut = 128;   // (the single-query byte-table scan: configuration 3 asks for k = 100)
constexpr int kRowLadderSearches = 64;   // searches that keep to the row-level ladder after the floorless level failed
bool first_level_is_best_of_block(const tv_index *ix, const SampledPlan &plan, size_t k_floor) {
    if (ix->row_ladder_left != 0) return false;
    if (effective_mode(ix) != TV_SCORE_P) return plan.lut_single && k_floor <= kBestLevelMaxKLut;   // u8 LUT: the single-query byte-table scan has the mode
    if (k_floor > kBestLevelMaxK) return false;
    return plan.wide ? tv::wide_serves_best_of_block(ix->geo.nch) : plan.nt_batched == 0;
}
SamplingSteps level_strides(const tv_index *ix, const SampledPlan &plan, size_t n_blocks, size_t k_floor, bool repeat) {
    if (!repeat && first_level_is_best_of_block(ix, plan, k_floor)) {
        SamplingSteps steps;
        // (the all-queries kernel pays for every candidate of the full scan -- a tile with one in it
        // leaves the integer fast path -- and samples twice as many blocks for a floor that lets half
        // as many through: 10M x 1536, 1024 queries: two rounds of its grid instead of one, +0.12 ms
        // of sampling, -0.25 ms of scan)
        const size_t per = plan.wide ? 1024 : 2048;
        size_t sample = std::max<size_t>((n_blocks * k_floor + per - 1) / per, 8 * k_floor);
        sample = std::min<size_t>(sample, size_t(plan.grid) * (tv::kSegCap / 2));   // a workgroup's blocks fit its segment
        size_t step = sample ? n_blocks / sample : 0;
        if (plan.wide) {
            // the all-queries-per-pass kernel works through the blocks in rounds of its grid and a
            // level costs whole rounds: trimmed to whole rounds, at least one, and never spilling into another
            const size_t round = size_t(plan.grid) * tv::wide_blocks_per_workgroup(ix->geo.nch);
            if (sample > round) sample -= sample % round;
            step = sample >= round ? (n_blocks + sample - 1) / sample : n_blocks / sample;
        }
        if (sample * 4 <= n_blocks && step > 1) {
            steps.step[steps.count++] = uint32_t(step);
            steps.step[steps.count++] = 1;
            steps.best_first = true;
            return steps;
        }
        // (an index too small for that level -- it would read a quarter of it or more -- takes the
        // row-level ladder below: a full scan from open floors alone would append every row)
    }
    // (the sixteen-query LUT scan works in rounds too: every wave of the grid carries two blocks through the row)
    return plan.wide    ? sampling_steps(n_blocks, k_floor, size_t(plan.grid) * tv::wide_blocks_per_workgroup(ix->geo.nch))
           : plan.lut16 ? sampling_steps(n_blocks, k_floor, size_t(plan.grid) * tv::lut16_blocks_per_workgroup(effective_mode(ix) == TV_SCORE_L_CLASSIC))
                        : sampling_steps(n_blocks, k_floor);
}
// Block offset of a repeated pass's level of stride `step`: it samples other blocks than the pass
// that misjudged the floor, half a stride in (an even number of blocks, so that mask words stay
// aligned).
uint32_t repeat_offset(uint32_t step) { return step >= 4 ? (step / 2) & ~1u : 0u; }

// The seam: search::search over device-resident inputs and outputs.
//
// Sample-then-filter.  Scans run in append mode: every allowed slot whose score
// reaches the query's floor is appended to a small per-query buffer, and a sort
// of that buffer yields either the next floor (sampling levels) or the answer
// (the full scan).  A floor is the k-th best score among slots actually
// scanned, hence a lower bound of the true k-th best, so the full scan appends
// every member of the true top-k; ties at the floor are kept (>=) and resolved
// by the same total order as everywhere else.
int search_device(tv_index *ix, const float *d_queries, size_t nq, size_t k, const uint64_t *d_mask,
                  size_t n_allowed, float *d_out_scores, int64_t *d_out_idx, size_t *out_k_eff) {
    const size_t n = ix->n;
    size_t k_eff = std::min(std::min(k, n), n_allowed);  // lib.rs:1460, search.rs:3222-3225
    if (out_k_eff) *out_k_eff = k_eff;
    ix->last_scan_ms = 0.0f;
    ix->last_scan_launches = 0;
    if (k_eff == 0 || nq == 0) return TV_OK;                // search.rs:3226-3229
    if (n >= (size_t(1) << 31)) { g_last_error = "index too large for 31-bit slots"; return TV_ERR_BAD_ARGUMENT; }
    const tv::Geometry &g = ix->geo;
    const int mode = effective_mode(ix);
    if (mode == TV_SCORE_P && g.bits != 4) { g_last_error = "score mode P needs 4-bit codes"; return TV_ERR_BAD_ARGUMENT; }
    const bool mode_p = mode == TV_SCORE_P;
    // a search on a lent, fixed workspace (tv_search_dev_noalloc) creates nothing, event pool included
    const bool timing = !ix->ws_fixed;
    int rc = timing ? ensure_events(ix) : TV_OK;
    if (rc != TV_OK) return rc;
    if (k_eff > size_t(tv::kMaxSampledK) || ix->force_robust)
        return search_robust(ix, d_queries, nq, k_eff, d_mask, d_out_scores, d_out_idx, timing);

    const size_t n_blocks = (n + tv::kVecBlock - 1) / tv::kVecBlock;
    // sampling levels take the k_floor-th best as the floor: a deeper order statistic is steadier
    const size_t k_floor = std::max<size_t>(k_eff, 16);
    if (ix->row_ladder_left > 0) --ix->row_ladder_left;
    if (ix->floorless_kept_left > 0) --ix->floorless_kept_left;
    uint32_t *h_over = ix->h_flags;   // pinned, one flag per query of a group, then the groups' level flags
    const bool track_levels = ix->track_levels != 0;
    // sized once for the whole call, repeated passes included: nothing is reallocated while work is in flight
    rc = ensure_workspace(ix, sampled_need_worst(ix, nq));
    if (rc != TV_OK) return rc;

    for (size_t g0 = 0; g0 < nq; g0 += kGroupQueries) {
        const size_t gq = std::min(kGroupQueries, nq - g0);
        Arena head;
        head.base = static_cast<uint8_t *>(ix->ws);
        int *d_raise = head.take<int>(gq);
        // The overflow flags of the first passes are written by k_final straight into the pinned
        // host array (device-visible): no copy kernel between the last selection and the host's read.
        uint32_t *d_over_all = ix->d_flags_host;
        head.take<uint32_t>(gq);
        uint32_t *d_rows = head.take<uint32_t>(std::min(gq, kWideChunkQueries));
        float *d_redo_q = head.take<float>(std::min(gq, kWideChunkQueries) * g.dim);
        // the group's chunks: (first query, relative to the group; length)
        size_t chunk_at[kGroupQueries / kChunkQueries + 1], n_chunks = 0;
        for (size_t c0 = 0; c0 < gq; c0 += chunk_len(ix, gq - c0)) chunk_at[n_chunks++] = c0;
        chunk_at[n_chunks] = gq;
        uint32_t *d_level_flags_all = head.take<uint32_t>(kLevelFlagWords);
        size_t n_timed = 0;

        // One pass over `pq_n` queries of the chunk at q0: the ladder from open floors, or, for the
        // packed batch of queries to repeat (rows d_rows[row0 ..]), the ladder again from the floors
        // the pass before raised for them.  Enqueues only; the caller synchronises.
        auto pass = [&](size_t q0, size_t row0, size_t pq_n, bool repeat, bool timed_pass, size_t chunk_no) -> int {
            const float *d_q = d_queries + q0 * g.dim;
            float *d_os = d_out_scores + q0 * k_eff;
            int64_t *d_oi = d_out_idx + q0 * k_eff;
            const SampledPlan plan = sampled_plan(ix, pq_n);
            const size_t tile_q = plan.tile_q, n_tiles = plan.n_tiles, cq_pad = plan.cq_pad, seg_stride = plan.seg_stride;
            const bool wide = plan.wide;
            const int grid = plan.grid;
            const SamplingSteps steps = level_strides(ix, plan, n_blocks, k_floor, repeat);
            const bool best_first = steps.best_first;
            uint32_t *d_level_flags = d_level_flags_all + chunk_no * SamplingSteps::kMax;
            if (head.used + plan.need > ix->ws_bytes) {
                g_last_error = "internal: workspace smaller than the pass it was sized for";
                return TV_ERR_BAD_ARGUMENT;
            }
            Arena ar;
            ar.base = static_cast<uint8_t *>(ix->ws) + head.used;
            int *d_tau = ar.take<int>(n_tiles * tv::kQTile);
            if (repeat) {
                TV_HIP(tv::launch_gather_redo(d_q, d_rows + row0, d_raise + (q0 - g0), g.dim, int(tile_q), pq_n, d_redo_q, d_tau,
                                              ix->stream));
                // every level of a repeated pass filters by a floor: all of their flags start at zero
                TV_HIP(tv::launch_fill_i32(reinterpret_cast<int *>(d_level_flags), 0, SamplingSteps::kMax, ix->stream));
            }
            Prepared pq;
            const int nt_batched = plan.nt_batched;
            int prc = prepare_queries(ix, ar, repeat ? d_redo_q : d_q, pq_n, pq,
                                      wide ? tv::wide_weights_split(g.nch) : (nt_batched == 0 || tv::batched_weights_split(g.nch)), false, true);
            if (prc != TV_OK) return prc;
            uint64_t *d_cand = ar.take<uint64_t>(cq_pad * seg_stride * tv::kSegCap);
            uint32_t *d_cnt = ar.take<uint32_t>(cq_pad * seg_stride);
            uint32_t *d_over = repeat ? ar.take<uint32_t>(cq_pad) : d_over_all + (q0 - g0);
            // no per-search clears: the first level reads the index's standing array of open floors,
            // every later one the floors k_final wrote, and k_final writes every overflow flag

            const int bgrid = tv::batched_grid_blocks(ix->device, g.nch);
            const bool batched = nt_batched > 0 && !wide;
            const size_t tiles_per_launch = wide ? n_tiles : batched ? size_t(nt_batched) : 1;
            if (!repeat && q0 == 0) ix->last_queries_per_launch = int(std::min(pq_n, tile_q * tiles_per_launch));   // the call's first chunk
            for (size_t lv = 0; lv < steps.size(); ++lv) {
                const bool last = lv + 1 == steps.size();
                // Sampling levels only yield floors, never slots, so the shifted origin of a repeated
                // pass needs no correction downstream.
                const uint32_t off = repeat ? repeat_offset(steps[lv]) : 0u;
                const size_t level_blocks = (n_blocks - off + steps[lv] - 1) / steps[lv];
                // level 1 appends every slot it reads: two blocks per workgroup fill a segment exactly
                const int lgrid = int(std::min<size_t>(size_t(grid), std::max<size_t>(1, (level_blocks + 1) / 2)));
                // A sampling level behind the first filters by the floor of the level before; when
                // that floor was far too low (rows laid out against the sample) its candidates do not
                // fit, k_final says so in the level's flag, and the level runs once more from the
                // floor k_final took from what did fit -- launches that do nothing unless the flag
                // is set.  The full scan then starts from the floor the level was meant to give.
                uint32_t *lv_flag = (!last && (lv > 0 || repeat)) ? d_level_flags + lv : nullptr;
                uint32_t *next_flag = (lv + 2 < steps.size()) ? d_level_flags + lv + 1 : nullptr;
                for (int attempt = 0; attempt < (lv_flag ? 2 : 1); ++attempt) {
                    const uint32_t *run_if = attempt == 0 ? nullptr : lv_flag;
                    int n_seg = lgrid;
                    size_t launch_no = 0;
                    // sampling levels of the sixteen-query LUT scan: all the chunk's tiles it serves in one
                    // launch, side by side (one tile leaves most of the chip idle for a round's time)
                    const size_t side_by_side = (plan.lut16 && !last && pq.d_tables16 != nullptr)
                                                    ? pq_n / tile_q + (pq_n % tile_q >= size_t(kLut16MinQueries) ? 1 : 0) : 0;
                    for (size_t t = 0; t < n_tiles; t += (t < side_by_side ? side_by_side : tiles_per_launch), ++launch_no) {
                        tv::ScanArgs a;
                        fill_scan_args(ix, a);
                        a.mask = d_mask;
                        a.tables = pq.d_tables + t * (mode_p ? pq.table_bytes_per_tile : tile_q * size_t(g.nch) * 1024);
                        a.qscale = pq.d_qscale + t * tile_q;
                        a.qbias = pq.d_qbias + t * tile_q;
                        a.nq_tile = int(std::min<size_t>(tile_q * tiles_per_launch, pq_n - t * tile_q));
                        a.k = 1;
                        a.gtau = ((lv == 0 && !repeat) ? ix->d_tau_open : d_tau) + t * tv::kQTile;
                        a.b_step = steps[lv];
                        a.run_if = run_if;
                        a.best_of_block = (best_first && lv == 0) ? 1 : 0;
                        if (off) {
                            a.codes += size_t(off) * g.block_bytes();
                            a.scales += size_t(off) * tv::kVecBlock;
                            if (a.mask) a.mask += off / 2;
                            a.n_blocks -= off;
                            a.n -= off * tv::kVecBlock;
                        }
                        a.cand = d_cand + t * tile_q * seg_stride * tv::kSegCap;
                        a.cand_cnt = d_cnt + t * tile_q * seg_stride;
                        a.seg_stride = uint32_t(seg_stride);
                        const bool timed = timed_pass && last && int(launch_no) < kMaxTimedTiles;
                        if (timed) TV_HIP(hipEventRecord(ix->ev_start[launch_no], ix->stream));
                        if (wide) {
                            n_seg = grid;
                            TV_HIP(tv::launch_scan_p4_wide(a, n_seg, ix->stream));
                        } else if (batched) {
                            n_seg = int(std::min<size_t>(size_t(bgrid), seg_stride));
                            TV_HIP(tv::launch_scan_p4_batched(a, n_seg, ix->stream));
                        } else if (mode_p) {
                            TV_HIP(tv::launch_scan_p4(a, lgrid, (best_first && lv == 0) ? tv::kModeBest : tv::kModeAppend, ix->stream));
                        } else if (t < side_by_side) {
                            a.tables = pq.d_tables16;
                            a.nq_tile = int(std::min<size_t>(pq_n, side_by_side * tile_q));
                            TV_HIP(tv::launch_scan_lut16(a, lgrid, int(side_by_side), ix->stream));
                        } else if (pq.d_tables16 != nullptr && a.nq_tile >= kLut16MinQueries) {
                            a.tables = pq.d_tables16 + t * tv::lut16_table_bytes(g.nch, tile_q);
                            TV_HIP(tv::launch_scan_lut16(a, lgrid, 1, ix->stream));
                        } else {
                            TV_HIP(tv::launch_scan_lut(a, lgrid, tv::kModeAppend, ix->stream));
                        }
                        if (timed) TV_HIP(hipEventRecord(ix->ev_stop[launch_no], ix->stream));
                    }
                    if (last && timed_pass) n_timed = std::min<size_t>(launch_no, size_t(kMaxTimedTiles));
                    // the first final pass may hand raised floors to a repeated one; the repeated pass
                    // sends what still does not fit to the exact path
                    TV_HIP(tv::launch_final(d_cand, d_cnt, uint32_t(n_seg), uint32_t(seg_stride), int(k_eff), int(k_floor),
                                            int(pq_n), d_os, d_oi, d_over, last ? nullptr : d_tau, int(tile_q),
                                            (lv > 0 || repeat) ? 1 : 0, (last && !repeat) ? d_raise + (q0 - g0) : nullptr,
                                            repeat ? d_rows + row0 : nullptr, lv_flag, attempt == 0 ? next_flag : nullptr,
                                            run_if, ix->stream));
                }
            }
            if (repeat) TV_HIP(hipMemcpyAsync(h_over, d_over, pq_n * sizeof(uint32_t), hipMemcpyDeviceToHost, ix->stream));
            return TV_OK;
        };

        // first passes of every chunk of the group, back to back; one read of the flags at the end
        for (size_t c = 0; c < n_chunks; ++c) {
            rc = pass(g0 + chunk_at[c], 0, chunk_at[c + 1] - chunk_at[c], false, timing && c == 0, c);
            if (rc != TV_OK) return rc;
        }
        if (track_levels)
            TV_HIP(hipMemcpyAsync(h_over + kGroupQueries, d_level_flags_all, kLevelFlagWords * 4, hipMemcpyDeviceToHost, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
        if (track_levels) {
            // flags of levels the passes above did not use hold whatever the workspace held: count only the used ones
            for (size_t c = 0; c < n_chunks; ++c) {
                const SampledPlan plan = sampled_plan(ix, chunk_at[c + 1] - chunk_at[c]);
                const size_t n_levels = level_strides(ix, plan, n_blocks, k_floor, false).size();
                for (size_t lv = 1; lv + 1 < n_levels; ++lv)
                    ix->level_repeats += h_over[kGroupQueries + c * SamplingSteps::kMax + lv] != 0u;
            }
        }
        for (size_t t = 0; t < n_timed; ++t) {
            float ms = 0.0f;
            TV_HIP(hipEventElapsedTime(&ms, ix->ev_start[t], ix->ev_stop[t]));
            ix->last_scan_ms += ms;
            ix->last_scan_launches += 1;
        }
        // Queries whose candidates did not fit (an unlucky sample, adversarial order).  Those that
        // came back with a raised floor (flag 1) are packed and scanned once more, a chunk's worth
        // together; what still does not fit then, and what had no floor to raise (flag 2), is
        // redone exactly.
        std::vector<uint32_t> redo_rows, exact_rows;    // group-relative query numbers
        for (size_t q = 0; q < gq; ++q) {
            if (h_over[q] == 1u) redo_rows.push_back(uint32_t(q));
            else if (h_over[q] != 0u) exact_rows.push_back(uint32_t(q));
        }
        ix->overflow_redos += redo_rows.size() + exact_rows.size();
        if ((redo_rows.size() + exact_rows.size()) * 8 >= gq) {
            if (level_strides(ix, sampled_plan(ix, chunk_at[1] - chunk_at[0]), n_blocks, k_floor, false).best_first) {
                // from here on, the repeated passes below included -- unless the row-level ladder has just failed too
                if (ix->floorless_kept_left == 0) ix->row_ladder_left = kRowLadderSearches;
            } else if (ix->row_ladder_left > 0) {
                // rows laid out against the row-level ladder as well: back to the floorless level, whose
                // failure is the cheaper one (its full scan gives up within a few rounds), and no
                // switching for a while
                ix->row_ladder_left = 0;
                ix->floorless_kept_left = kRowLadderSearches;
            }
        }
        const size_t room = ix->ws_bytes - head.used;
        for (size_t i = 0; i < redo_rows.size();) {
            // rows of one chunk go together: all of them in one pass when the workspace holds that
            // pass, else in the largest pieces it holds
            size_t chunk = 0;
            while (chunk_at[chunk + 1] <= redo_rows[i]) ++chunk;
            size_t e = i;
            while (e < redo_rows.size() && redo_rows[e] < chunk_at[chunk + 1]) ++e;
            size_t piece = std::min<size_t>(e - i, tv::kQTile);
            for (size_t cand_piece : kRepeatPieces) {
                const size_t m = std::min(cand_piece, e - i);
                if (sampled_plan(ix, m).need <= room) { piece = m; break; }
            }
            for (size_t r = 0; r < piece; ++r) h_over[r] = redo_rows[i + r] - uint32_t(chunk_at[chunk]);   // pinned staging
            TV_HIP(hipMemcpyAsync(d_rows, h_over, piece * sizeof(uint32_t), hipMemcpyHostToDevice, ix->stream));
            TV_HIP(hipStreamSynchronize(ix->stream));
            rc = pass(g0 + chunk_at[chunk], 0, piece, true, false, chunk);
            if (rc != TV_OK) return rc;
            TV_HIP(hipStreamSynchronize(ix->stream));
            for (size_t r = 0; r < piece; ++r)
                if (h_over[r] != 0u) exact_rows.push_back(redo_rows[i + r]);
            i += piece;
        }
        std::sort(exact_rows.begin(), exact_rows.end());
        ix->exact_redos += exact_rows.size();
        for (size_t i = 0; i < exact_rows.size();) {
            size_t e = i + 1;
            while (e < exact_rows.size() && exact_rows[e] == exact_rows[e - 1] + 1) ++e;     // runs of neighbours go together
            const size_t qa = g0 + exact_rows[i], cnt = e - i;
            rc = search_robust(ix, d_queries + qa * g.dim, cnt, k_eff, d_mask, d_out_scores + qa * k_eff, d_out_idx + qa * k_eff,
                               false);
            if (rc != TV_OK) return rc;
            i = e;
        }
    }
    return TV_OK;
}

// ---- search calls, merged ----------------------------------------------------------------------
// The reference's search takes &self and runs on as many caller threads as there are
// (turbovec/src/lib.rs:22-52, tests/concurrent_search.rs); one GPU serves one launch at a time, and a
// launch costs the same for one query as for thirty-two.  So calls do not queue up one behind the
// other: a call registers itself, then waits for the index; whoever gets it next serves every
// registered call that is compatible with its own (same kind of buffers, same k, same mask) as one
// batch -- rows of a batch are scored independently, so each caller receives exactly what a call of
// its own would have returned -- and the others find their results ready when their turn comes.
constexpr size_t kMergeQueries = 4096;   // queries one merged batch may hold

}  // namespace

struct tv_request {
    bool host = true;              // tv_search (host buffers) or tv_search_dev (device buffers)
    const float *q = nullptr;
    size_t nq = 0, k = 0;
    const uint64_t *mask = nullptr;
    size_t mask_arg = 0;           // host: number of mask words; device: the mask's popcount
    float *out_s = nullptr;
    int64_t *out_i = nullptr;
    size_t k_eff = 0;
    int rc = TV_OK;
    std::string err;
    bool done = false;
};

namespace {

// Serves the calls of `batch` (compatible with each other, at least one) as one search.  The index
// lock is held.  Returns the status every one of them gets.
int serve_batch(tv_index *ix, const std::vector<tv_request *> &batch, size_t *k_eff_out) {
    const tv_request &r0 = *batch[0];
    TV_HIP(hipSetDevice(ix->device));
    const size_t n = ix->n, dim = size_t(ix->geo.dim);
    size_t nq = 0;
    for (const tv_request *r : batch) nq += r->nq;
    if (!r0.host) {
        const size_t n_allowed = r0.mask ? r0.mask_arg : n;
        if (batch.size() == 1)
            return search_device(ix, r0.q, nq, r0.k, r0.mask, n_allowed, r0.out_s, r0.out_i, k_eff_out);
        // several callers' device buffers: gathered into the staging allocation, results scattered back
        const size_t k_eff = std::min(std::min(r0.k, n), n_allowed);
        *k_eff_out = k_eff;
        if (k_eff == 0 || nq == 0) return TV_OK;
        const size_t q_bytes = round_up(nq * dim * sizeof(float), 256), s_bytes = round_up(nq * k_eff * sizeof(float), 256);
        const size_t i_bytes = round_up(nq * k_eff * sizeof(int64_t), 256);
        int rc = ensure_io(ix, q_bytes + s_bytes + i_bytes);
        if (rc != TV_OK) return rc;
        uint8_t *base = static_cast<uint8_t *>(ix->io);
        float *d_q = reinterpret_cast<float *>(base);
        float *d_s = reinterpret_cast<float *>(base + q_bytes);
        int64_t *d_i = reinterpret_cast<int64_t *>(base + q_bytes + s_bytes);
        size_t at = 0;
        for (const tv_request *r : batch) {
            if (r->nq) TV_HIP(hipMemcpyAsync(d_q + at * dim, r->q, r->nq * dim * sizeof(float), hipMemcpyDeviceToDevice, ix->stream));
            at += r->nq;
        }
        rc = search_device(ix, d_q, nq, r0.k, r0.mask, n_allowed, d_s, d_i, nullptr);
        if (rc != TV_OK) return rc;
        at = 0;
        for (const tv_request *r : batch) {
            if (r->nq) {
                TV_HIP(hipMemcpyAsync(r->out_s, d_s + at * k_eff, r->nq * k_eff * sizeof(float), hipMemcpyDeviceToDevice, ix->stream));
                TV_HIP(hipMemcpyAsync(r->out_i, d_i + at * k_eff, r->nq * k_eff * sizeof(int64_t), hipMemcpyDeviceToDevice, ix->stream));
            }
            at += r->nq;
        }
        TV_HIP(hipStreamSynchronize(ix->stream));
        return TV_OK;
    }
    const uint64_t *mask_words = r0.mask;
    const size_t n_mask_words = r0.mask_arg;
    size_t n_allowed = n;
    if (mask_words) {
        if (n_mask_words != (n + 63) / 64) return TV_ERR_MASK_LENGTH_MISMATCH;
        n_allowed = 0;  // search.rs:3222-3225; bits at or past n are ignored
        for (size_t w = 0; w < n_mask_words; ++w) {
            uint64_t word = mask_words[w];
            if (w * 64 + 64 > n) word &= (n - w * 64 >= 64) ? ~uint64_t(0) : ((uint64_t(1) << (n - w * 64)) - 1);
            n_allowed += size_t(__builtin_popcountll(word));
        }
    }
    const size_t k_eff = std::min(std::min(r0.k, n), n_allowed);
    *k_eff_out = k_eff;
    ix->last_scan_ms = 0.0f;
    ix->last_scan_launches = 0;
    if (k_eff == 0 || nq == 0) return TV_OK;
    // host staging: queries, mask and results live in the index's own staging allocation (kept
    // between calls, so a search allocates nothing once it has seen its largest batch), apart
    // from the per-chunk workspace, which is re-carved freely
    const size_t q_bytes = round_up(nq * dim * sizeof(float), 256), s_bytes = round_up(nq * k_eff * sizeof(float), 256);
    const size_t i_bytes = round_up(nq * k_eff * sizeof(int64_t), 256), m_bytes = mask_words ? round_up(n_mask_words * 8, 256) : 0;
    int rc = ensure_io(ix, q_bytes + s_bytes + i_bytes + m_bytes);
    if (rc != TV_OK) return rc;
    uint8_t *base = static_cast<uint8_t *>(ix->io);
    float *d_q = reinterpret_cast<float *>(base);
    float *d_s = reinterpret_cast<float *>(base + q_bytes);
    int64_t *d_i = reinterpret_cast<int64_t *>(base + q_bytes + s_bytes);
    uint64_t *d_m = mask_words ? reinterpret_cast<uint64_t *>(base + q_bytes + s_bytes + i_bytes) : nullptr;
    size_t at = 0;
    for (const tv_request *r : batch) {
        if (r->nq && hipMemcpyAsync(d_q + at * dim, r->q, r->nq * dim * sizeof(float), hipMemcpyHostToDevice, ix->stream) != hipSuccess) {
            g_last_error = "host to device copy failed";
            return TV_ERR_HIP;
        }
        at += r->nq;
    }
    if (mask_words && hipMemcpyAsync(d_m, mask_words, n_mask_words * 8, hipMemcpyHostToDevice, ix->stream) != hipSuccess) {
        g_last_error = "host to device copy failed";
        return TV_ERR_HIP;
    }
    rc = search_device(ix, d_q, nq, r0.k, d_m, n_allowed, d_s, d_i, nullptr);
    if (rc != TV_OK) return rc;
    at = 0;
    for (const tv_request *r : batch) {
        if (r->nq && (hipMemcpyAsync(r->out_s, d_s + at * k_eff, r->nq * k_eff * sizeof(float), hipMemcpyDeviceToHost, ix->stream) != hipSuccess ||
                      hipMemcpyAsync(r->out_i, d_i + at * k_eff, r->nq * k_eff * sizeof(int64_t), hipMemcpyDeviceToHost, ix->stream) != hipSuccess)) {
            g_last_error = "device to host copy failed";
            return TV_ERR_HIP;
        }
        at += r->nq;
    }
    if (hipStreamSynchronize(ix->stream) != hipSuccess) {
        g_last_error = "device to host copy failed";
        return TV_ERR_HIP;
    }
    return TV_OK;
}

bool compatible(const tv_request &a, const tv_request &b) {
    return a.host == b.host && a.k == b.k && a.mask == b.mask && a.mask_arg == b.mask_arg;
}

// How long a caller that is about to serve waits for the callers of the batch before to come back
// with their next call (they were all released at the same moment and are a few microseconds of
// host code away from asking again).  Only after a batch that did merge calls.
constexpr auto kGatherWait = std::chrono::microseconds(300);

int search_merged(tv_index *ix, tv_request &r) {
    std::vector<tv_request *> batch;
    {
        std::unique_lock<std::mutex> reg(ix->waiting_mu);
        ix->waiting.push_back(&r);
        ix->waiting_cv.notify_all();       // a serving caller gathering its batch may be waiting for this one
        for (;;) {
            if (r.done) {                  // served by another caller's launch
                if (r.rc != TV_OK) g_last_error = r.err;
                return r.rc;
            }
            if (!ix->serving) break;
            ix->waiting_cv.wait(reg);
        }
        ix->serving = true;
        // Callers in a loop come back together: when the batch before held several calls, give the
        // same number a moment to register again instead of serving this one alone and all of them
        // in the launch after.
        if (ix->last_batch_calls > 1) {
            const auto deadline = std::chrono::steady_clock::now() + kGatherWait;
            while (ix->waiting.size() < ix->last_batch_calls)
                if (ix->waiting_cv.wait_until(reg, deadline) == std::cv_status::timeout) break;
        }
        // this call first, then the compatible ones in order of arrival, up to the batch limit
        batch.push_back(&r);
        size_t total = r.nq;
        std::vector<tv_request *> rest;
        for (tv_request *w : ix->waiting) {
            if (w == &r) continue;
            if (compatible(*w, r) && total + w->nq <= kMergeQueries) { batch.push_back(w); total += w->nq; }
            else rest.push_back(w);
        }
        ix->waiting.swap(rest);
    }
    size_t k_eff = 0;
    int rc;
    {
        std::lock_guard<std::mutex> lock(ix->mu);   // against the entry points that change the index
        g_last_error.clear();
        rc = serve_batch(ix, batch, &k_eff);
    }
    {
        std::lock_guard<std::mutex> reg(ix->waiting_mu);
        for (tv_request *w : batch) {
            w->rc = rc;
            w->k_eff = k_eff;
            if (rc != TV_OK) w->err = g_last_error;
            w->done = true;
        }
        ix->merged_calls += batch.size() - 1;
        ix->last_batch_calls = batch.size();
        ix->serving = false;
    }
    ix->waiting_cv.notify_all();
    return rc;
}

}  // namespace

extern "C" {

const char *tv_status_string(int status) {
    switch (status) {
        case TV_OK: return "ok";
        case TV_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM: return "query buffer length not a multiple of dim";
        case TV_ERR_INVALID_QUERY_VALUE: return "invalid query value (must be finite and |value| < 1e16)";
        case TV_ERR_MASK_LENGTH_MISMATCH: return "mask length does not match index size";
        case TV_ERR_ALLOWLIST_EMPTY: return "allowlist is empty";
        case TV_ERR_UNKNOWN_ID: return "id in allowlist is not present in index";
        case TV_ERR_BAD_ARGUMENT: return "bad argument";
        case TV_ERR_HIP: return "HIP runtime error";
        case TV_ERR_NO_DEVICE: return "no usable GPU";
        case TV_ERR_INDEX_OUT_OF_RANGE: return "index out of range";
        case TV_ERR_BAD_IMAGE: return "invalid snapshot image";
        default: return "unknown status";
    }
}

const char *tv_last_error(void) { return g_last_error.c_str(); }

int tv_index_create(int dim, int bits, int device, tv_index **out) {
    if (!out) return TV_ERR_BAD_ARGUMENT;
    *out = nullptr;
    if (bits < 2 || bits > 4) { g_last_error = "bit_width must be 2, 3, or 4"; return TV_ERR_BAD_ARGUMENT; }
    if (dim <= 0 || dim % 8 != 0) { g_last_error = "dim must be a positive multiple of 8"; return TV_ERR_BAD_ARGUMENT; }
    if (dim > 16384) { g_last_error = "dim exceeds maximum 16384"; return TV_ERR_BAD_ARGUMENT; }
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= device || device < 0) {
        g_last_error = "no HIP device with that ordinal";
        return TV_ERR_NO_DEVICE;
    }
    TV_HIP(hipSetDevice(device));
    tv_index *ix = new (std::nothrow) tv_index();
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    ix->device = device;
    ix->geo.dim = dim;
    ix->geo.bits = bits;
    ix->geo.G = dim / (8 / bits);
    ix->geo.nch = (ix->geo.G + tv::kChunkGroups - 1) / tv::kChunkGroups;
    // 4-bit rows are padded with whole chunks of zero groups (their query weights are zero, so they
    // add nothing) up to a chunk count the all-queries-per-pass kernel has an instance for: even
    // from 9 chunks on, a multiple of 4 above 24, of 8 above 48 (to 96 chunks = 6144 dimensions).
    // The padding is part of the resident index on every path: at most 3 chunks (of 25: +12 %), 7
    // (of 49: +14 %), one in seven at worst; the device block is geo.block_bytes() = nch * 1024
    // bytes, not ceil(G / 32) * 1024.
    if (bits == 4 && ix->geo.nch >= 9) {
        if (ix->geo.nch > 48 && ix->geo.nch <= 96) ix->geo.nch = (ix->geo.nch + 7) / 8 * 8;
        else if (ix->geo.nch > 24 && ix->geo.nch <= 48) ix->geo.nch = (ix->geo.nch + 3) / 4 * 4;
        else if (ix->geo.nch <= 24) ix->geo.nch += ix->geo.nch & 1;
    }
    ix->rot = tv::make_rotation_tables(dim);
    ix->cb = tv::make_codebook(bits, dim);
    derive_levels(ix);
    int rc = TV_OK;
    do {
        if (hipStreamCreateWithFlags(&ix->stream, hipStreamNonBlocking) != hipSuccess) { rc = TV_ERR_HIP; break; }
        if (hipMalloc(reinterpret_cast<void **>(&ix->d_signs), 2 * size_t(dim) * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&ix->d_perms), 2 * size_t(dim) * sizeof(uint32_t)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&ix->d_centroids), 16 * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&ix->d_tq_shift), size_t(dim) * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&ix->d_tq_scale), size_t(dim) * sizeof(float)) != hipSuccess ||
            hipMalloc(reinterpret_cast<void **>(&ix->d_tau_open), kTauOpenInts * sizeof(int)) != hipSuccess) {
            rc = TV_ERR_HIP;
            break;
        }
        if (hipHostMalloc(reinterpret_cast<void **>(&ix->h_flags), (kGroupQueries + kLevelFlagWords) * sizeof(uint32_t), hipHostMallocMapped) != hipSuccess) {
            rc = TV_ERR_HIP;
            break;
        }
        if (hipHostGetDevicePointer(reinterpret_cast<void **>(&ix->d_flags_host), ix->h_flags, 0) != hipSuccess) {
            rc = TV_ERR_HIP;
            break;
        }
        rc = scratch_address(device, &ix->scratch);
        if (rc != TV_OK) break;
        // floors of a search's first sampling level: the order key of -inf for every query, written once
        if (tv::launch_fill_i32(ix->d_tau_open, int(0x807fffffu), kTauOpenInts, ix->stream) != hipSuccess ||
            hipStreamSynchronize(ix->stream) != hipSuccess) {
            rc = TV_ERR_HIP;
            break;
        }
        rc = upload_tables(ix);
    } while (0);
    if (rc != TV_OK) {
        if (g_last_error.empty()) g_last_error = "device allocation failed";
        tv_index_destroy(ix);
        return rc;
    }
    *out = ix;
    return TV_OK;
}

int tv_index_destroy(tv_index *ix) {
    if (!ix) return TV_OK;
    (void)hipSetDevice(ix->device);
    if (ix->stream) (void)hipStreamSynchronize(ix->stream);
    void *ptrs[] = {ix->d_signs, ix->d_perms, ix->d_centroids, ix->d_tq_shift, ix->d_tq_scale,
                    ix->d_codes, ix->d_scales, ix->ws, ix->io, ix->d_tau_open};
    for (void *p : ptrs) if (p) (void)hipFree(p);
    if (ix->h_flags) (void)hipHostFree(ix->h_flags);
    if (ix->events_ready)
        for (int i = 0; i < tv::kTimedLaunches; ++i) {
            (void)hipEventDestroy(ix->ev_start[i]);
            (void)hipEventDestroy(ix->ev_stop[i]);
        }
    if (ix->stream) (void)hipStreamDestroy(ix->stream);
    delete ix;
    return TV_OK;
}

int tv_index_set_tables(tv_index *ix, const float *signs, const uint32_t *perms, const float *centroids) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    const size_t dim = size_t(ix->geo.dim);
    if (signs) ix->rot.signs.assign(signs, signs + 2 * dim);
    if (perms) {
        for (size_t i = 0; i < 2 * dim; ++i) if (perms[i] >= dim) return TV_ERR_BAD_ARGUMENT;
        ix->rot.perms.assign(perms, perms + 2 * dim);
    }
    if (centroids) {
        ix->cb.centroids.assign(centroids, centroids + (size_t(1) << ix->geo.bits));
        for (size_t i = 0; i + 1 < ix->cb.centroids.size(); ++i)
            ix->cb.boundaries[i] = (ix->cb.centroids[i] + ix->cb.centroids[i + 1]) * 0.5f;
        derive_levels(ix);
    }
    return upload_tables(ix);
}

int tv_index_set_calibration(tv_index *ix, const float *shift, const float *scale) {
    if (!ix || (shift == nullptr) != (scale == nullptr)) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    const size_t dim = size_t(ix->geo.dim);
    if (!shift) { ix->tq_shift.clear(); ix->tq_scale.clear(); return TV_OK; }
    ix->tq_shift.assign(shift, shift + dim);
    ix->tq_scale.assign(scale, scale + dim);
    TV_HIP(hipMemcpyAsync(ix->d_tq_shift, shift, dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
    TV_HIP(hipMemcpyAsync(ix->d_tq_scale, scale, dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    return TV_OK;
}

int tv_index_set_score_mode(tv_index *ix, int mode) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    if (mode != TV_SCORE_AUTO && mode != TV_SCORE_L_SCALAR && mode != TV_SCORE_L_CLASSIC && mode != TV_SCORE_L_U32 && mode != TV_SCORE_P)
        return TV_ERR_BAD_ARGUMENT;
    if (mode == TV_SCORE_P && ix->geo.bits != 4) { g_last_error = "score mode P needs 4-bit codes"; return TV_ERR_BAD_ARGUMENT; }
    std::lock_guard<std::mutex> lock(ix->mu);
    ix->score_mode = mode;
    return TV_OK;
}

int tv_index_get_tables(const tv_index *ix, float *signs, uint32_t *perms, float *centroids, float *boundaries) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    if (signs) std::memcpy(signs, ix->rot.signs.data(), ix->rot.signs.size() * sizeof(float));
    if (perms) std::memcpy(perms, ix->rot.perms.data(), ix->rot.perms.size() * sizeof(uint32_t));
    if (centroids) std::memcpy(centroids, ix->cb.centroids.data(), ix->cb.centroids.size() * sizeof(float));
    if (boundaries) std::memcpy(boundaries, ix->cb.boundaries.data(), ix->cb.boundaries.size() * sizeof(float));
    return TV_OK;
}

int tv_index_upload_seq(tv_index *ix, const uint8_t *seq_codes, size_t n_vectors, const float *scales) {
    if (!ix || (n_vectors && (!seq_codes || !scales))) return TV_ERR_BAD_ARGUMENT;
    if (n_vectors >= (size_t(1) << 31)) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    ix->n = 0;
    int rc = ensure_capacity(ix, n_vectors);
    if (rc != TV_OK) return rc;
    const tv::Geometry &g = ix->geo;
    const size_t n_blocks = (n_vectors + tv::kVecBlock - 1) / tv::kVecBlock;
    const size_t seq_block = size_t(g.G) * tv::kVecBlock;
    rc = clear_tail_blocks(ix, n_blocks);
    if (rc != TV_OK) return rc;
    // stage the sequential-blocked bytes through the workspace in slices
    const size_t slice_blocks = std::max<size_t>(1, (size_t(256) << 20) / seq_block);
    rc = ensure_workspace(ix, std::min(n_blocks, slice_blocks) * seq_block + 256);
    if (rc != TV_OK) return rc;
    for (size_t b0 = 0; b0 < n_blocks; b0 += slice_blocks) {
        const size_t nb = std::min(slice_blocks, n_blocks - b0);
        TV_HIP(hipMemcpyAsync(ix->ws, seq_codes + b0 * seq_block, nb * seq_block, hipMemcpyHostToDevice, ix->stream));
        TV_HIP(tv::launch_seq_to_native(static_cast<const uint8_t *>(ix->ws), ix->d_codes, g, b0, nb, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
    }
    if (n_vectors) {
        TV_HIP(hipMemsetAsync(ix->d_scales, 0, n_blocks * tv::kVecBlock * sizeof(float), ix->stream));
        TV_HIP(hipMemcpyAsync(ix->d_scales, scales, n_vectors * sizeof(float), hipMemcpyHostToDevice, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
    }
    ix->n = n_vectors;
    return TV_OK;
}

int tv_index_upload_seq_dev(tv_index *ix, const uint8_t *d_seq_codes, size_t n_vectors, const float *d_scales) {
    if (!ix || (n_vectors && (!d_seq_codes || !d_scales))) return TV_ERR_BAD_ARGUMENT;
    if (n_vectors >= (size_t(1) << 31)) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    ix->n = 0;
    int rc = ensure_capacity(ix, n_vectors);
    if (rc != TV_OK) return rc;
    const size_t n_blocks = (n_vectors + tv::kVecBlock - 1) / tv::kVecBlock;
    const size_t seq_block = size_t(ix->geo.G) * tv::kVecBlock;
    rc = clear_tail_blocks(ix, n_blocks);
    if (rc != TV_OK) return rc;
    const size_t slice_blocks = std::max<size_t>(1, (size_t(1) << 30) / seq_block);  // keeps each grid small
    for (size_t b0 = 0; b0 < n_blocks; b0 += slice_blocks) {
        const size_t nb = std::min(slice_blocks, n_blocks - b0);
        TV_HIP(tv::launch_seq_to_native(d_seq_codes + b0 * seq_block, ix->d_codes, ix->geo, b0, nb, ix->stream));
    }
    if (n_vectors) {
        TV_HIP(hipMemsetAsync(ix->d_scales, 0, n_blocks * tv::kVecBlock * sizeof(float), ix->stream));
        TV_HIP(hipMemcpyAsync(ix->d_scales, d_scales, n_vectors * sizeof(float), hipMemcpyDeviceToDevice, ix->stream));
    }
    TV_HIP(hipStreamSynchronize(ix->stream));
    ix->n = n_vectors;
    return TV_OK;
}

int tv_index_append_rows(tv_index *ix, const uint8_t *rows, const float *scales, size_t n_new) {
    if (!ix || (n_new && (!rows || !scales))) return TV_ERR_BAD_ARGUMENT;
    if (n_new == 0) return TV_OK;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    if (ix->n + n_new >= (size_t(1) << 31)) return TV_ERR_BAD_ARGUMENT;
    int rc = ensure_capacity(ix, ix->n + n_new);
    if (rc != TV_OK) return rc;
    const tv::Geometry &g = ix->geo;
    const size_t slice = std::max<size_t>(1, (size_t(64) << 20) / size_t(g.G));
    rc = ensure_workspace(ix, std::min(n_new, slice) * size_t(g.G) + 256);
    if (rc != TV_OK) return rc;
    for (size_t r0 = 0; r0 < n_new; r0 += slice) {
        const size_t nr = std::min(slice, n_new - r0);
        TV_HIP(hipMemcpyAsync(ix->ws, rows + r0 * g.G, nr * size_t(g.G), hipMemcpyHostToDevice, ix->stream));
        TV_HIP(tv::launch_append_rows(static_cast<const uint8_t *>(ix->ws), ix->d_codes, g, ix->n + r0, nr, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
    }
    TV_HIP(hipMemcpyAsync(ix->d_scales + ix->n, scales, n_new * sizeof(float), hipMemcpyHostToDevice, ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    ix->n += n_new;
    return TV_OK;
}

// lib.rs add -> encode.rs:1418-1476 on the device, then append_lanes (pack.rs:211-233).
static int add_device_rows(tv_index *ix, const float *d_vectors, size_t n_new) {
    const tv::Geometry &g = ix->geo;
    const bool cal = !ix->tq_shift.empty();
    const size_t slice = size_t(1) << 20;
    for (size_t r0 = 0; r0 < n_new; r0 += slice) {
        const size_t nr = std::min(slice, n_new - r0);
        TV_HIP(tv::launch_encode(d_vectors + r0 * size_t(g.dim), nr, ix->n + r0, ix->d_signs, ix->d_perms,
                                 cal ? ix->d_tq_shift : nullptr, cal ? ix->d_tq_scale : nullptr,
                                 ix->cb.centroids.data(), ix->cb.boundaries.data(), g, ix->rot.block,
                                 ix->rot.inv_sqrt_block, ix->d_codes, ix->d_scales, nullptr, ix->stream));
    }
    TV_HIP(hipStreamSynchronize(ix->stream));
    ix->n += n_new;
    return TV_OK;
}

int tv_index_add_dev(tv_index *ix, const float *d_vectors, size_t n_new) {
    if (!ix || (n_new && !d_vectors)) return TV_ERR_BAD_ARGUMENT;
    if (n_new == 0) return TV_OK;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    if (ix->n + n_new >= (size_t(1) << 31)) return TV_ERR_BAD_ARGUMENT;
    int rc = ensure_capacity(ix, ix->n + n_new);
    if (rc != TV_OK) return rc;
    return add_device_rows(ix, d_vectors, n_new);
}

int tv_index_add(tv_index *ix, const float *vectors, size_t n_new) {
    if (!ix || (n_new && !vectors)) return TV_ERR_BAD_ARGUMENT;
    if (n_new == 0) return TV_OK;
    const size_t dim = size_t(ix->geo.dim);
    size_t bad = 0;
    int rc = tv_validate_queries(vectors, n_new * dim, ix->geo.dim, &bad);   // same predicate, encode.rs:76-83
    if (rc != TV_OK) {
        g_last_error = "vector " + std::to_string(bad / dim) + " holds a non-finite or too large value";
        return rc;
    }
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    if (ix->n + n_new >= (size_t(1) << 31)) return TV_ERR_BAD_ARGUMENT;
    rc = ensure_capacity(ix, ix->n + n_new);
    if (rc != TV_OK) return rc;
    const size_t slice = std::max<size_t>(1, (size_t(256) << 20) / (dim * sizeof(float)));
    rc = ensure_workspace(ix, std::min(n_new, slice) * dim * sizeof(float) + 256);
    if (rc != TV_OK) return rc;
    for (size_t r0 = 0; r0 < n_new; r0 += slice) {
        const size_t nr = std::min(slice, n_new - r0);
        TV_HIP(hipMemcpyAsync(ix->ws, vectors + r0 * dim, nr * dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
        rc = add_device_rows(ix, static_cast<const float *>(ix->ws), nr);
        if (rc != TV_OK) return rc;
    }
    return TV_OK;
}

// TurboQuantIndex::calibrate (lib.rs:2599) on an empty index: rotate the normalised sample on
// the device (encode.rs:406-458), fit on the host (encode.rs:737-857), commit the pair.
int tv_index_calibrate(tv_index *ix, const float *sample, size_t n) {
    if (!ix || !sample) return TV_ERR_BAD_ARGUMENT;
    if (n < 2) { g_last_error = "calibration needs at least 2 rows"; return TV_ERR_BAD_ARGUMENT; }   // encode.rs:395
    const size_t dim = size_t(ix->geo.dim);
    size_t bad = 0;
    int rc = tv_validate_queries(sample, n * dim, ix->geo.dim, &bad);
    if (rc != TV_OK) {
        g_last_error = "sample row " + std::to_string(bad / dim) + " holds a non-finite or too large value";
        return rc;
    }
    std::vector<float> rotated(n * dim);
    {
        std::lock_guard<std::mutex> lock(ix->mu);
        if (ix->n != 0) {
            g_last_error = "calibrate on a populated index (re-encoding stored rows) is not supported";
            return TV_ERR_BAD_ARGUMENT;
        }
        TV_HIP(hipSetDevice(ix->device));
        const size_t slice = std::max<size_t>(1, (size_t(128) << 20) / (dim * sizeof(float)));
        rc = ensure_workspace(ix, 2 * std::min(n, slice) * dim * sizeof(float) + 512);
        if (rc != TV_OK) return rc;
        float *d_in = static_cast<float *>(ix->ws);
        float *d_out = d_in + std::min(n, slice) * dim;
        for (size_t r0 = 0; r0 < n; r0 += slice) {
            const size_t nr = std::min(slice, n - r0);
            TV_HIP(hipMemcpyAsync(d_in, sample + r0 * dim, nr * dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
            TV_HIP(tv::launch_encode(d_in, nr, 0, ix->d_signs, ix->d_perms, nullptr, nullptr, ix->cb.centroids.data(),
                                     ix->cb.boundaries.data(), ix->geo, ix->rot.block, ix->rot.inv_sqrt_block,
                                     nullptr, nullptr, d_out, ix->stream));
            TV_HIP(hipMemcpyAsync(rotated.data() + r0 * dim, d_out, nr * dim * sizeof(float), hipMemcpyDeviceToHost, ix->stream));
            TV_HIP(hipStreamSynchronize(ix->stream));
        }
    }
    std::vector<float> shift(dim), scale(dim);
    tv::fit_tqplus(rotated.data(), n, ix->geo.dim, ix->cb.centroids, shift.data(), scale.data());
    return tv_index_set_calibration(ix, shift.data(), scale.data());
}

int tv_index_get_calibration(const tv_index *ix, float *shift, float *scale, size_t *n_calib) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    if (n_calib) *n_calib = ix->tq_shift.size();
    if (shift && !ix->tq_shift.empty()) std::memcpy(shift, ix->tq_shift.data(), ix->tq_shift.size() * sizeof(float));
    if (scale && !ix->tq_scale.empty()) std::memcpy(scale, ix->tq_scale.data(), ix->tq_scale.size() * sizeof(float));
    return TV_OK;
}

int tv_index_swap_remove(tv_index *ix, size_t idx) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    if (idx >= ix->n) return TV_ERR_INDEX_OUT_OF_RANGE;
    TV_HIP(hipSetDevice(ix->device));
    TV_HIP(tv::launch_move_lane(ix->d_codes, ix->d_scales, ix->geo, ix->n - 1, idx, ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    ix->n -= 1;
    return TV_OK;
}

// The index's lock is held by the caller.
static int download_seq_locked(tv_index *ix, uint8_t *seq_out, float *scales_out) {
    TV_HIP(hipSetDevice(ix->device));
    const tv::Geometry &g = ix->geo;
    const size_t n_blocks = (ix->n + tv::kVecBlock - 1) / tv::kVecBlock;
    const size_t seq_block = size_t(g.G) * tv::kVecBlock;
    if (seq_out && n_blocks) {
        const size_t slice_blocks = std::max<size_t>(1, (size_t(256) << 20) / seq_block);
        int rc = ensure_workspace(ix, std::min(n_blocks, slice_blocks) * seq_block + 256);
        if (rc != TV_OK) return rc;
        for (size_t b0 = 0; b0 < n_blocks; b0 += slice_blocks) {
            const size_t nb = std::min(slice_blocks, n_blocks - b0);
            TV_HIP(tv::launch_native_to_seq(ix->d_codes, static_cast<uint8_t *>(ix->ws), g, b0, nb, ix->stream));
            TV_HIP(hipMemcpyAsync(seq_out + b0 * seq_block, ix->ws, nb * seq_block, hipMemcpyDeviceToHost, ix->stream));
            TV_HIP(hipStreamSynchronize(ix->stream));
        }
    }
    if (scales_out && ix->n) {
        TV_HIP(hipMemcpyAsync(scales_out, ix->d_scales, ix->n * sizeof(float), hipMemcpyDeviceToHost, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
    }
    return TV_OK;
}

int tv_index_download_seq(const tv_index *cix, uint8_t *seq_out, float *scales_out) {
    tv_index *ix = const_cast<tv_index *>(cix);
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    return download_seq_locked(ix, seq_out, scales_out);
}

size_t tv_index_len(const tv_index *ix) { return ix ? ix->n : 0; }
int tv_index_dim(const tv_index *ix) { return ix ? ix->geo.dim : 0; }
int tv_index_bits(const tv_index *ix) { return ix ? ix->geo.bits : 0; }

int tv_validate_queries(const float *queries, size_t len, int dim, size_t *bad_index) {
    if (dim <= 0 || len % size_t(dim) != 0) return TV_ERR_QUERY_BUFFER_NOT_MULTIPLE_OF_DIM;
    for (size_t i = 0; i < len; ++i) {
        if (!(std::fabs(queries[i]) < 1e16f)) {
            if (bad_index) *bad_index = i;
            return TV_ERR_INVALID_QUERY_VALUE;
        }
    }
    return TV_OK;
}

int tv_pack_mask(const uint8_t *mask_bytes, size_t n, uint64_t *words_out, size_t *n_allowed) {
    if ((n && !mask_bytes) || !words_out) return TV_ERR_BAD_ARGUMENT;
    size_t allowed = 0;
    for (size_t w = 0; w * 64 < n; ++w) {
        uint64_t word = 0;
        const size_t lim = std::min<size_t>(64, n - w * 64);
        for (size_t bit = 0; bit < lim; ++bit) word |= uint64_t(mask_bytes[w * 64 + bit] != 0) << bit;
        allowed += size_t(__builtin_popcountll(word));
        words_out[w] = word;
    }
    if (n_allowed) *n_allowed = allowed;
    return TV_OK;
}

int tv_search_dev(tv_index *ix, const float *d_queries, size_t nq, size_t k, const uint64_t *d_mask_words,
                  size_t n_allowed, float *d_out_scores, int64_t *d_out_indices, size_t *out_k_eff) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    tv_request r;
    r.host = false;
    r.q = d_queries; r.nq = nq; r.k = k;
    r.mask = d_mask_words; r.mask_arg = d_mask_words ? n_allowed : 0;
    r.out_s = d_out_scores; r.out_i = d_out_indices;
    const int rc = search_merged(ix, r);
    if (out_k_eff) *out_k_eff = r.k_eff;
    return rc;
}

size_t tv_noalloc_scratch_bytes(void) { return kScratchBytes; }

int tv_search_dev_noalloc(tv_index *ix, const float *d_queries, size_t nq, size_t k, const uint64_t *d_mask_words,
                          size_t n_allowed, float *d_out_scores, int64_t *d_out_indices, size_t *out_k_eff) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    if (!d_mask_words) n_allowed = ix->n;
    const size_t k_eff = std::min(std::min(k, ix->n), n_allowed);
    // What the search may carve, worst case: the sampled path's chunk, and the exact path a query
    // falls back to when its candidates overflow.  Refused up front when that exceeds the array.
    size_t need = 0;
    if (k_eff != 0 && nq != 0) {
        const size_t cq = std::min(nq, kChunkQueries);    // the exact path works in chunks of this size throughout
        need = robust_need(ix, cq, k_eff);
        if (k_eff <= size_t(tv::kMaxSampledK) && !ix->force_robust) need = std::max(need, sampled_need_worst(ix, nq));
    }
    if (need > kScratchBytes) {
        g_last_error = "tv_search_dev_noalloc: " + std::to_string(nq) + " queries, k=" + std::to_string(k) + " over " +
                       std::to_string(ix->n) + " rows may need " + std::to_string(need) +
                       " bytes of scratch; the fixed buffer holds " + std::to_string(kScratchBytes) +
                       " (fewer queries per call; k <= 32 on a large index)";
        return TV_ERR_BAD_ARGUMENT;
    }
    std::lock_guard<std::mutex> device_lock(g_scratch[ix->device].in_use);
    void *own_ws = ix->ws;
    const size_t own_bytes = ix->ws_bytes;
    ix->ws = ix->scratch;
    ix->ws_bytes = kScratchBytes;
    ix->ws_fixed = true;
    const int rc = search_device(ix, d_queries, nq, k, d_mask_words, n_allowed, d_out_scores, d_out_indices, out_k_eff);
    ix->ws = own_ws;
    ix->ws_bytes = own_bytes;
    ix->ws_fixed = false;
    return rc;
}

int tv_search(tv_index *ix, const float *queries, size_t nq, size_t k, const uint64_t *mask_words,
              size_t n_mask_words, float *out_scores, int64_t *out_indices, size_t *out_k_eff) {
    if (!ix || (nq && !queries)) return TV_ERR_BAD_ARGUMENT;
    tv_request r;
    r.host = true;
    r.q = queries; r.nq = nq; r.k = k;
    r.mask = mask_words; r.mask_arg = mask_words ? n_mask_words : 0;
    r.out_s = out_scores; r.out_i = out_indices;
    const int rc = search_merged(ix, r);
    if (out_k_eff) *out_k_eff = r.k_eff;
    return rc;
}

int tv_debug_scan(tv_index *ix, const float *queries, size_t nq, int32_t *acc_out, float *scores_out) {
    if (!ix || (nq && !queries)) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    const size_t n = ix->n;
    if (n == 0 || nq == 0) return TV_OK;
    const tv::Geometry &g = ix->geo;
    const int mode = effective_mode(ix);
    const bool mode_p = mode == TV_SCORE_P;
    const size_t tile_q = mode_p ? size_t(tv::kQTile) : size_t(lut_tile_q(ix, 1));
    for (size_t q0 = 0; q0 < nq; q0 += tile_q) {
        const size_t cq = std::min<size_t>(tile_q, nq - q0);
        size_t need = prepare_bytes(ix, cq) + round_up(cq * g.dim * 4, 256) + 2 * round_up(cq * n * 4, 256) + 65536;
        int rc = ensure_workspace(ix, need);
        if (rc != TV_OK) return rc;
        Arena ar;
        ar.base = static_cast<uint8_t *>(ix->ws);
        float *d_q = ar.take<float>(cq * g.dim);
        int32_t *d_acc = ar.take<int32_t>(cq * n);
        float *d_sc = ar.take<float>(cq * n);
        TV_HIP(hipMemcpyAsync(d_q, queries + q0 * g.dim, cq * g.dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
        Prepared pq;
        rc = prepare_queries(ix, ar, d_q, cq, pq);
        if (rc != TV_OK) return rc;
        tv::ScanArgs a;
        fill_scan_args(ix, a);
        a.tables = pq.d_tables;
        a.qscale = pq.d_qscale;
        a.qbias = pq.d_qbias;
        a.nq_tile = int(cq);
        a.k = 1;
        a.acc_out = d_acc;
        a.score_out = d_sc;
        const int grid = tv::scan_grid_blocks(ix->device, mode_p, g.nch, 1, int(tile_q));
        if (mode_p) TV_HIP(tv::launch_scan_p4(a, grid, tv::kModeDump, ix->stream));
        else TV_HIP(tv::launch_scan_lut(a, grid, tv::kModeDump, ix->stream));
        if (acc_out) TV_HIP(hipMemcpyAsync(acc_out + q0 * n, d_acc, cq * n * 4, hipMemcpyDeviceToHost, ix->stream));
        if (scores_out) TV_HIP(hipMemcpyAsync(scores_out + q0 * n, d_sc, cq * n * 4, hipMemcpyDeviceToHost, ix->stream));
        TV_HIP(hipStreamSynchronize(ix->stream));
    }
    return TV_OK;
}

int tv_debug_prepare(tv_index *ix, const float *queries, size_t nq, float *q_rot_out, float *scale_out,
                     float *bias_out) {
    if (!ix || (nq && !queries)) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    if (nq == 0) return TV_OK;
    const tv::Geometry &g = ix->geo;
    int rc = ensure_workspace(ix, prepare_bytes(ix, nq) + round_up(nq * g.dim * 4, 256) + 65536);
    if (rc != TV_OK) return rc;
    Arena ar;
    ar.base = static_cast<uint8_t *>(ix->ws);
    float *d_q = ar.take<float>(nq * g.dim);
    TV_HIP(hipMemcpyAsync(d_q, queries, nq * g.dim * sizeof(float), hipMemcpyHostToDevice, ix->stream));
    Prepared pq;
    rc = prepare_queries(ix, ar, d_q, nq, pq, true, true);
    if (rc != TV_OK) return rc;
    if (q_rot_out) TV_HIP(hipMemcpyAsync(q_rot_out, pq.d_qrot, nq * g.dim * 4, hipMemcpyDeviceToHost, ix->stream));
    if (scale_out) TV_HIP(hipMemcpyAsync(scale_out, pq.d_qscale, nq * 4, hipMemcpyDeviceToHost, ix->stream));
    if (bias_out) TV_HIP(hipMemcpyAsync(bias_out, pq.d_qbias, nq * 4, hipMemcpyDeviceToHost, ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    return TV_OK;
}

int tv_host_rotation_tables(int dim, float *signs, uint32_t *perms, int *block, float *inv_sqrt_block) {
    if (dim <= 0 || dim % 8 != 0 || dim > 16384) return TV_ERR_BAD_ARGUMENT;
    const tv::RotationTables t = tv::make_rotation_tables(dim);
    if (signs) std::memcpy(signs, t.signs.data(), t.signs.size() * sizeof(float));
    if (perms) std::memcpy(perms, t.perms.data(), t.perms.size() * sizeof(uint32_t));
    if (block) *block = t.block;
    if (inv_sqrt_block) *inv_sqrt_block = t.inv_sqrt_block;
    return TV_OK;
}

int tv_host_codebook(int bits, int dim, float *boundaries, float *centroids) {
    if (bits < 2 || bits > 4 || dim < 8 || dim > 16384) return TV_ERR_BAD_ARGUMENT;
    const tv::Codebook cb = tv::make_codebook(bits, dim);
    if (boundaries) std::memcpy(boundaries, cb.boundaries.data(), cb.boundaries.size() * sizeof(float));
    if (centroids) std::memcpy(centroids, cb.centroids.data(), cb.centroids.size() * sizeof(float));
    return TV_OK;
}

size_t tv_host_snapshot_len(int format, int dim, int bits, int kind, size_t n_calib, size_t n) {
    if (format != 6 && format != 7) return 0;
    return tv::snapshot_len(format, dim, bits, kind, n_calib, n);
}

int tv_host_snapshot_compose(int format, int dim, int bits, int kind, const float *boundaries, const float *centroids,
                             size_t n_calib, const float *shift, const float *scale,
                             const uint8_t *seq, size_t n, const float *scales, const uint64_t *ids,
                             uint8_t *out) {
    if (format != 6 && format != 7) return TV_ERR_BAD_ARGUMENT;
    if (bits < 2 || bits > 4 || dim <= 0 || dim % 8 != 0 || dim > 16384 || kind < 0 || kind > 1) return TV_ERR_BAD_ARGUMENT;
    if (!boundaries || !centroids || !out || (n && (!seq || !scales)) || (kind == 1 && n && !ids)) return TV_ERR_BAD_ARGUMENT;
    if ((n_calib != 0 && n_calib != size_t(dim)) || (n_calib && (!shift || !scale))) return TV_ERR_BAD_ARGUMENT;
    const tv::SnapshotParts s{kind, dim, bits, boundaries, centroids, n_calib, shift, scale, seq, n, scales, ids};
    tv::snapshot_compose(format, s, out);
    return TV_OK;
}

int tv_host_snapshot_info(const uint8_t *bytes, size_t len, int *format, int *kind, int *dim, int *bits,
                          size_t *n_calib, size_t *n) {
    if (!bytes) return TV_ERR_BAD_ARGUMENT;
    tv::SnapshotInfo info;
    const std::string why = tv::snapshot_parse(bytes, len, info);
    if (!why.empty()) { g_last_error = why; return TV_ERR_BAD_IMAGE; }
    if (format) *format = info.format;
    if (kind) *kind = info.kind;
    if (dim) *dim = info.dim;
    if (bits) *bits = info.bits;
    if (n_calib) *n_calib = info.n_calib;
    if (n) *n = info.n;
    return TV_OK;
}

int tv_host_snapshot_extract(const uint8_t *bytes, size_t len, float *boundaries, float *centroids,
                             float *shift, float *scale, uint8_t *seq, float *scales, uint64_t *ids) {
    if (!bytes) return TV_ERR_BAD_ARGUMENT;
    tv::SnapshotInfo info;
    const std::string why = tv::snapshot_parse(bytes, len, info);
    if (!why.empty()) { g_last_error = why; return TV_ERR_BAD_IMAGE; }
    const size_t nl = size_t(1) << info.bits;
    if (boundaries) std::memcpy(boundaries, bytes + info.boundaries_at, (nl - 1) * 4);
    if (centroids) std::memcpy(centroids, bytes + info.centroids_at, nl * 4);
    if (shift) std::memcpy(shift, bytes + info.shift_at, info.n_calib * 4);
    if (scale) std::memcpy(scale, bytes + info.scale_at, info.n_calib * 4);
    if (seq || scales || ids) {
        const size_t nb = (info.n + 31) / 32;
        std::vector<uint8_t> seq_tmp;
        std::vector<float> sc_tmp;
        if (!seq) { seq_tmp.resize(nb * info.row_bytes * 32); seq = seq_tmp.data(); }
        if (!scales) { sc_tmp.resize(nb * 32); scales = sc_tmp.data(); }
        tv::snapshot_extract(bytes, info, seq, scales, ids);
    }
    return TV_OK;
}

int tv_index_to_bytes(const tv_index *cix, const uint64_t *ids, int format, uint8_t *out, size_t cap, size_t *len) {
    tv_index *ix = const_cast<tv_index *>(cix);
    if (!ix || !len || (format != 6 && format != 7)) return TV_ERR_BAD_ARGUMENT;
    const int kind = ids ? 1 : 0;
    // one lock over size, download and compose: the image is of one state of the index
    std::lock_guard<std::mutex> lock(ix->mu);
    const size_t n = ix->n, n_calib = ix->tq_shift.size();
    *len = tv::snapshot_len(format, ix->geo.dim, ix->geo.bits, kind, n_calib, n);
    if (!out) return TV_OK;
    if (cap < *len) return TV_ERR_BAD_ARGUMENT;
    const size_t nb = (n + 31) / 32;
    std::vector<uint8_t> seq(nb * size_t(ix->geo.G) * 32);
    std::vector<float> scales(n);
    int rc = download_seq_locked(ix, seq.data(), scales.data());
    if (rc != TV_OK) return rc;
    const tv::SnapshotParts s{kind, ix->geo.dim, ix->geo.bits, ix->cb.boundaries.data(), ix->cb.centroids.data(),
                              n_calib, ix->tq_shift.data(), ix->tq_scale.data(), seq.data(), n, scales.data(), ids};
    tv::snapshot_compose(format, s, out);
    return TV_OK;
}

int tv_index_from_bytes(const uint8_t *bytes, size_t len, int device, tv_index **out, uint64_t *ids_out) {
    if (!bytes || !out) return TV_ERR_BAD_ARGUMENT;
    *out = nullptr;
    tv::SnapshotInfo info;
    const std::string why = tv::snapshot_parse(bytes, len, info);
    if (!why.empty()) { g_last_error = why; return TV_ERR_BAD_IMAGE; }
    tv_index *ix = nullptr;
    int rc = tv_index_create(info.dim, info.bits, device, &ix);
    if (rc != TV_OK) return rc;
    const size_t nl = size_t(1) << info.bits;
    std::vector<float> cen(nl), sh(info.n_calib), sc(info.n_calib);
    std::memcpy(cen.data(), bytes + info.centroids_at, nl * 4);
    std::memcpy(sh.data(), bytes + info.shift_at, info.n_calib * 4);
    std::memcpy(sc.data(), bytes + info.scale_at, info.n_calib * 4);
    rc = tv_index_set_tables(ix, nullptr, nullptr, cen.data());
    if (rc == TV_OK && info.n_calib) rc = tv_index_set_calibration(ix, sh.data(), sc.data());
    if (rc == TV_OK && info.n) {
        const size_t nb = (info.n + 31) / 32;
        std::vector<uint8_t> seq(nb * info.row_bytes * 32);
        std::vector<float> scales(nb * 32);
        tv::snapshot_extract(bytes, info, seq.data(), scales.data(), ids_out);
        rc = tv_index_upload_seq(ix, seq.data(), info.n, scales.data());
    }
    if (rc != TV_OK) { tv_index_destroy(ix); return rc; }
    *out = ix;
    return TV_OK;
}

int tv_debug_stream_probe(tv_index *ix, const void *d_src, void *d_dst, size_t bytes, int reps, float *ms_per_rep) {
    if (!ix || !d_src || reps <= 0) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    int rc = ensure_events(ix);
    if (rc != TV_OK) return rc;
    rc = ensure_workspace(ix, 4096);
    if (rc != TV_OK) return rc;
    uint32_t *sink = static_cast<uint32_t *>(ix->ws);
    TV_HIP(tv::launch_probe(d_src, d_dst, bytes, d_dst != nullptr, sink, ix->stream));  // warm
    TV_HIP(hipEventRecord(ix->ev_start[0], ix->stream));
    for (int r = 0; r < reps; ++r) TV_HIP(tv::launch_probe(d_src, d_dst, bytes, d_dst != nullptr, sink, ix->stream));
    TV_HIP(hipEventRecord(ix->ev_stop[0], ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    float ms = 0.0f;
    TV_HIP(hipEventElapsedTime(&ms, ix->ev_start[0], ix->ev_stop[0]));
    if (ms_per_rep) *ms_per_rep = ms / float(reps);
    return TV_OK;
}

int tv_debug_mfma_probe(tv_index *ix, int iters, int reps, float *ms_per_rep, double *ops_per_rep) {
    if (!ix || iters <= 0 || reps <= 0) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    TV_HIP(hipSetDevice(ix->device));
    int rc = ensure_events(ix);
    if (rc != TV_OK) return rc;
    rc = ensure_workspace(ix, 4096);
    if (rc != TV_OK) return rc;
    uint32_t *sink = static_cast<uint32_t *>(ix->ws);
    double ops = 0.0;
    TV_HIP(tv::launch_probe_mfma(ix->device, iters, sink, &ops, ix->stream));  // warm
    TV_HIP(hipEventRecord(ix->ev_start[0], ix->stream));
    for (int r = 0; r < reps; ++r) TV_HIP(tv::launch_probe_mfma(ix->device, iters, sink, &ops, ix->stream));
    TV_HIP(hipEventRecord(ix->ev_stop[0], ix->stream));
    TV_HIP(hipStreamSynchronize(ix->stream));
    float ms = 0.0f;
    TV_HIP(hipEventElapsedTime(&ms, ix->ev_start[0], ix->ev_stop[0]));
    if (ms_per_rep) *ms_per_rep = ms / float(reps);
    if (ops_per_rep) *ops_per_rep = ops;
    return TV_OK;
}

int tv_debug_set_path(tv_index *ix, int force_full_lists) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    ix->force_robust = (force_full_lists & 1) != 0;
    ix->no_batched = (force_full_lists & 2) != 0;
    ix->no_wide = (force_full_lists & 4) != 0;
    ix->no_lut16 = (force_full_lists & 8) != 0;
    return TV_OK;
}

int tv_debug_sampling_plan(const tv_index *cix, size_t nq, size_t k, uint32_t *strides, uint32_t *repeat_offsets, size_t cap,
                           size_t *count) {
    tv_index *ix = const_cast<tv_index *>(cix);
    if (!ix || !count) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    *count = 0;
    const size_t k_eff = std::min(k, ix->n);
    if (k_eff == 0 || nq == 0 || k_eff > size_t(tv::kMaxSampledK) || ix->force_robust) return TV_OK;   // no ladder
    const size_t n_blocks = (ix->n + tv::kVecBlock - 1) / tv::kVecBlock;
    const SampledPlan plan = sampled_plan(ix, chunk_len(ix, nq));
    const SamplingSteps steps = level_strides(ix, plan, n_blocks, std::max<size_t>(k_eff, 16), false);
    *count = steps.size();
    for (size_t i = 0; i < steps.size() && i < cap; ++i) {
        if (strides) strides[i] = steps[i];
        if (repeat_offsets) repeat_offsets[i] = repeat_offset(steps[i]);
    }
    return TV_OK;
}

int tv_debug_level_repeats(tv_index *ix, int track, size_t *count) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    if (track >= 0) ix->track_levels = track;
    if (count) *count = ix->level_repeats;
    return TV_OK;
}

int tv_debug_workspace_bytes(const tv_index *cix, size_t *workspace, size_t *staging) {
    tv_index *ix = const_cast<tv_index *>(cix);
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ix->mu);
    if (workspace) *workspace = ix->ws_bytes;
    if (staging) *staging = ix->io_bytes;
    return TV_OK;
}

int tv_debug_overflow_redos(const tv_index *ix, size_t *count) {
    if (!ix || !count) return TV_ERR_BAD_ARGUMENT;
    *count = ix->overflow_redos;
    return TV_OK;
}

int tv_debug_exact_redos(const tv_index *ix, size_t *count) {
    if (!ix || !count) return TV_ERR_BAD_ARGUMENT;
    *count = ix->exact_redos;
    return TV_OK;
}

int tv_debug_merged_calls(const tv_index *cix, size_t *count) {
    tv_index *ix = const_cast<tv_index *>(cix);
    if (!ix || !count) return TV_ERR_BAD_ARGUMENT;
    std::lock_guard<std::mutex> reg(ix->waiting_mu);
    *count = ix->merged_calls;
    return TV_OK;
}

int tv_debug_queries_per_launch(const tv_index *ix, int *queries) {
    if (!ix || !queries) return TV_ERR_BAD_ARGUMENT;
    *queries = ix->last_queries_per_launch;
    return TV_OK;
}

int tv_last_scan_ms(const tv_index *ix, float *ms, int *launches) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    if (ms) *ms = ix->last_scan_ms;
    if (launches) *launches = ix->last_scan_launches;
    return TV_OK;
}

int tv_index_device_ptrs(const tv_index *ix, void **d_codes, void **d_scales, size_t *code_bytes) {
    if (!ix) return TV_ERR_BAD_ARGUMENT;
    if (d_codes) *d_codes = ix->d_codes;
    if (d_scales) *d_scales = ix->d_scales;
    if (code_bytes) *code_bytes = (ix->n + tv::kVecBlock - 1) / tv::kVecBlock * ix->geo.block_bytes();
    return TV_OK;
}

}  // extern "C"
