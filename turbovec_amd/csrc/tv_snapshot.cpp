// Snapshot images: the byte form TurboQuantIndex::to_bytes / IdMapIndex::to_bytes
// and `write` produce (turbovec/src/io_v7.rs), composed and parsed on the host
// from the sequential-blocked codes the device layout converts to and from.
//
// Layout of an unclaimed generation-0 image (io_v7.rs:902-925 write_image):
//   superblock   "TV7\0", version 2, bit_width u8, kind u8, dim u32, nonce u64 = 0,
//                MAX_OPS u32 = 1024, boundaries f32[], centroids f32[], n_calib u32,
//                shift f32[], scale f32[], CRC-32C                       (:516-542)
//   header A     gen u64 = 0, n u64, the n % 32 tail rows (G code bytes, scale f32,
//                id u64 for kind 1), 0 op groups u32, delta {0 materialised u32,
//                appended range 0..0 (2 x u32), digest u32}, CRC-32C, zero padding
//                up to the slot's fixed reserve                          (:549-599)
//   header B     all zero (invalid on purpose)
//   n / 32 units 32*G sequential-blocked code bytes, 32 scales, 32 ids   (:602-629)
// All integers and floats little-endian.
//
// The flat container the release before wrote (turbovec/src/convert.rs:14-31, :453-512), still
// what the reference's committed sha256 digests of to_bytes() hash, is handled too (format 6):
//   "TVPI" (kind 0) or "TVIM" (kind 1), version u8 = 6, bit_width u8, dim u32, n u64,
//   boundaries, centroids, sequential-blocked codes padded to whole blocks, n scales,
//   n_calib u32, shifts, scales, and for kind 1 n ids.  No checksums.
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "tv_snapshot.h"

namespace tv {

namespace {

constexpr size_t kBlock = 32;
constexpr uint32_t kMaxOps = 1024;     // io_v7.rs:117, a format constant
constexpr uint8_t kVersion = 2;        // io_v7.rs:101

const uint32_t *crc_table() {
    static uint32_t table[256];
    static bool ready = false;
    if (!ready) {
        for (uint32_t i = 0; i < 256; ++i) {
            uint32_t c = i;
            for (int k = 0; k < 8; ++k) c = (c >> 1) ^ (0x82F63B78u & (0u - (c & 1u)));   // Castagnoli, reflected
            table[i] = c;
        }
        ready = true;
    }
    return table;
}

uint32_t crc_update(uint32_t crc, const uint8_t *p, size_t n) {
    const uint32_t *t = crc_table();
    for (size_t i = 0; i < n; ++i) crc = (crc >> 8) ^ t[(crc ^ p[i]) & 0xffu];
    return crc;
}

uint32_t crc_one(const uint8_t *p, size_t n) { return ~crc_update(0xFFFFFFFFu, p, n); }

void put_u32(std::vector<uint8_t> &v, uint32_t x) { for (int i = 0; i < 4; ++i) v.push_back(uint8_t(x >> (8 * i))); }
void put_u64(std::vector<uint8_t> &v, uint64_t x) { for (int i = 0; i < 8; ++i) v.push_back(uint8_t(x >> (8 * i))); }
void put_f32(std::vector<uint8_t> &v, float f) { uint32_t x; std::memcpy(&x, &f, 4); put_u32(v, x); }
uint32_t get_u32(const uint8_t *p) { return uint32_t(p[0]) | uint32_t(p[1]) << 8 | uint32_t(p[2]) << 16 | uint32_t(p[3]) << 24; }
uint64_t get_u64(const uint8_t *p) { return uint64_t(get_u32(p)) | uint64_t(get_u32(p + 4)) << 32; }
float get_f32(const uint8_t *p) { const uint32_t x = get_u32(p); float f; std::memcpy(&f, &x, 4); return f; }

// io_v7.rs:283-335: a CRC over bytes that never sit contiguously, with the same length-derived
// three-way split as snapshot_crc32.
struct DeltaDigest {
    size_t at = 0, s1 = 0, s2 = 0;
    bool split = false;
    uint32_t parts[3] = {0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};
    explicit DeltaDigest(size_t total) {
        split = total >= 4096;
        if (split) { s1 = total / 3; s2 = s1 * 2; }
    }
    void push(const uint8_t *p, size_t n) {
        if (!split) { parts[0] = crc_update(parts[0], p, n); at += n; return; }
        while (n) {
            const int part = at < s1 ? 0 : (at < s2 ? 1 : 2);
            const size_t end = part == 0 ? s1 : (part == 1 ? s2 : SIZE_MAX);
            const size_t take = n < end - at ? n : end - at;
            parts[part] = crc_update(parts[part], p, take);
            at += take; p += take; n -= take;
        }
    }
    uint32_t finish() const {
        if (!split) return ~parts[0];
        uint8_t d[12];
        for (int i = 0; i < 3; ++i) { const uint32_t v = ~parts[i]; for (int b = 0; b < 4; ++b) d[i * 4 + b] = uint8_t(v >> (8 * b)); }
        return crc_one(d, 12);
    }
};

struct Geo {
    int kind, dim, bits;
    size_t n_calib;
    size_t row_bytes() const { return size_t(dim) / size_t(bits == 2 ? 4 : 2); }   // pack.rs:252-257
    size_t n_levels() const { return size_t(1) << bits; }
    size_t id_bytes(size_t rows) const { return kind == 1 ? rows * 8 : 0; }
    size_t sb_len() const { return 23 + (n_levels() - 1) * 4 + n_levels() * 4 + 4 + n_calib * 8 + 4; }   // io_v7.rs:380-382
    size_t op_size() const { return 1 + row_bytes() + 4 + id_bytes(1); }
    size_t hdr_len() const {                                                                            // io_v7.rs:409-417
        return 16 + 31 * (row_bytes() + 4 + id_bytes(1)) + 4 + kMaxOps * (5 + op_size()) + 4 + size_t(kMaxOps) * 4 + 12 + 4;
    }
    size_t unit_len() const { return kBlock * row_bytes() + kBlock * 4 + id_bytes(kBlock); }
    size_t unit_at(size_t block) const { return sb_len() + 2 * hdr_len() + block * unit_len(); }
};

}  // namespace

// io_v7.rs:128-141: inputs of 4096 bytes or more are checksummed as three thirds, and the value
// stored is the CRC of the three digests.
uint32_t snapshot_crc32(const uint8_t *p, size_t n) {
    if (n < 4096) return crc_one(p, n);
    const size_t third = n / 3;
    const uint32_t c[3] = {crc_one(p, third), crc_one(p + third, third), crc_one(p + 2 * third, n - 2 * third)};
    uint8_t d[12];
    for (int i = 0; i < 3; ++i) for (int b = 0; b < 4; ++b) d[i * 4 + b] = uint8_t(c[i] >> (8 * b));
    return crc_one(d, 12);
}

size_t snapshot_len(int format, int dim, int bits, int kind, size_t n_calib, size_t n) {
    const Geo g{kind, dim, bits, n_calib};
    if (format == 6) {
        const size_t nb = (n + kBlock - 1) / kBlock;
        return 18 + (2 * g.n_levels() - 1) * 4 + nb * g.row_bytes() * kBlock + n * 4 + 4 + n_calib * 8 + g.id_bytes(n);
    }
    return g.unit_at(n / kBlock);     // io_v7.rs:446-451 full_len
}

static void compose_flat6(const SnapshotParts &s, uint8_t *out) {
    const Geo g{s.kind, s.dim, s.bits, s.n_calib};
    std::vector<uint8_t> v;
    v.insert(v.end(), {'T', 'V', uint8_t(s.kind == 1 ? 'I' : 'P'), uint8_t(s.kind == 1 ? 'M' : 'I')});
    v.push_back(6);
    v.push_back(uint8_t(s.bits));
    put_u32(v, uint32_t(s.dim));
    put_u64(v, uint64_t(s.n));
    for (size_t i = 0; i + 1 < g.n_levels(); ++i) put_f32(v, s.boundaries[i]);
    for (size_t i = 0; i < g.n_levels(); ++i) put_f32(v, s.centroids[i]);
    uint8_t *p = out;
    std::memcpy(p, v.data(), v.size()); p += v.size();
    const size_t code_bytes = (s.n + kBlock - 1) / kBlock * g.row_bytes() * kBlock;
    if (code_bytes) std::memcpy(p, s.seq, code_bytes);
    p += code_bytes;
    v.clear();
    for (size_t i = 0; i < s.n; ++i) put_f32(v, s.scales[i]);
    put_u32(v, uint32_t(s.n_calib));
    for (size_t i = 0; i < s.n_calib; ++i) put_f32(v, s.shift[i]);
    for (size_t i = 0; i < s.n_calib; ++i) put_f32(v, s.scale[i]);
    if (s.kind == 1) for (size_t i = 0; i < s.n; ++i) put_u64(v, s.ids[i]);
    std::memcpy(p, v.data(), v.size());
}

void snapshot_compose(int format, const SnapshotParts &s, uint8_t *out) {
    if (format == 6) { compose_flat6(s, out); return; }
    const Geo g{s.kind, s.dim, s.bits, s.n_calib};
    const size_t G = g.row_bytes();
    std::vector<uint8_t> sb;
    sb.insert(sb.end(), {'T', 'V', '7', 0});
    sb.push_back(kVersion);
    sb.push_back(uint8_t(s.bits));
    sb.push_back(uint8_t(s.kind));
    put_u32(sb, uint32_t(s.dim));
    put_u64(sb, 0);                    // UNCLAIMED_NONCE: the bytes are a pure function of index state
    put_u32(sb, kMaxOps);
    for (size_t i = 0; i + 1 < g.n_levels(); ++i) put_f32(sb, s.boundaries[i]);
    for (size_t i = 0; i < g.n_levels(); ++i) put_f32(sb, s.centroids[i]);
    put_u32(sb, uint32_t(s.n_calib));
    for (size_t i = 0; i < s.n_calib; ++i) put_f32(sb, s.shift[i]);
    for (size_t i = 0; i < s.n_calib; ++i) put_f32(sb, s.scale[i]);
    put_u32(sb, snapshot_crc32(sb.data(), sb.size()));

    std::vector<uint8_t> h;
    put_u64(h, 0);                     // generation
    put_u64(h, uint64_t(s.n));
    const size_t n_tail = s.n % kBlock, first_tail = s.n - n_tail;
    for (size_t k = 0; k < n_tail; ++k) {
        const size_t r = first_tail + k, b = r / kBlock, lane = r % kBlock;
        for (size_t gi = 0; gi < G; ++gi) h.push_back(s.seq[(b * G + gi) * kBlock + lane]);   // lib.rs:1648-1675
        put_f32(h, s.scales[r]);
        if (s.kind == 1) put_u64(h, s.ids[r]);
    }
    put_u32(h, 0);                     // no pending op groups
    put_u32(h, 0);                     // delta: nothing materialised,
    put_u32(h, 0);                     //        appended range 0..0,
    put_u32(h, 0);
    {
        DeltaDigest d(8);              //        digest of the generation alone (io_v7.rs:819-831)
        const uint8_t gen[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        d.push(gen, 8);
        put_u32(h, d.finish());
    }
    put_u32(h, snapshot_crc32(h.data(), h.size()));

    uint8_t *p = out;
    std::memcpy(p, sb.data(), sb.size()); p += sb.size();
    std::memset(p, 0, 2 * g.hdr_len());
    std::memcpy(p, h.data(), h.size()); p += 2 * g.hdr_len();
    const size_t n_blocks = s.n / kBlock;
    for (size_t b = 0; b < n_blocks; ++b) {
        std::memcpy(p, s.seq + b * G * kBlock, G * kBlock); p += G * kBlock;
        for (size_t l = 0; l < kBlock; ++l) { uint32_t x; std::memcpy(&x, &s.scales[b * kBlock + l], 4); for (int i = 0; i < 4; ++i) *p++ = uint8_t(x >> (8 * i)); }
        if (s.kind == 1)
            for (size_t l = 0; l < kBlock; ++l) { const uint64_t x = s.ids[b * kBlock + l]; for (int i = 0; i < 8; ++i) *p++ = uint8_t(x >> (8 * i)); }
    }
}

// Parse and validate; on success fills `info` (offsets into `bytes`).  Returns an empty string
// or the reason the image is refused.
static std::string parse_flat6(const uint8_t *bytes, size_t len, SnapshotInfo &info) {
    if (len < 18) return "truncated image";
    if (bytes[4] != 6) return "flat container version " + std::to_string(bytes[4]) + " is not supported (6 is)";
    Geo g{};
    g.kind = bytes[2] == 'I' ? 1 : 0;
    g.bits = bytes[5];
    g.dim = int(get_u32(bytes + 6));
    const uint64_t n = get_u64(bytes + 10);
    if (g.bits < 2 || g.bits > 4) return "bit_width out of range";
    if (g.dim <= 0 || g.dim % 8 != 0 || g.dim > 16384) return "dim out of range";
    if (n >= (uint64_t(1) << 31)) return "row count out of range";
    const size_t nl = g.n_levels(), nb = (size_t(n) + kBlock - 1) / kBlock;
    const size_t codes_at = 18 + (2 * nl - 1) * 4;
    const size_t scales_at = codes_at + nb * g.row_bytes() * kBlock;
    const size_t calib_at = scales_at + size_t(n) * 4;
    if (len < calib_at + 4) return "truncated image";
    g.n_calib = get_u32(bytes + calib_at);
    if (g.n_calib != 0 && g.n_calib != size_t(g.dim)) return "calibration length is neither 0 nor dim";
    if (len != snapshot_len(6, g.dim, g.bits, g.kind, g.n_calib, size_t(n))) return "image length does not match its row count";
    info.format = 6; info.kind = g.kind; info.dim = g.dim; info.bits = g.bits; info.n_calib = g.n_calib; info.n = size_t(n);
    info.boundaries_at = 18; info.centroids_at = 18 + (nl - 1) * 4;
    info.shift_at = calib_at + 4; info.scale_at = calib_at + 4 + g.n_calib * 4;
    info.units_at = codes_at; info.tail_at = scales_at; info.unit_len = 0; info.row_bytes = g.row_bytes();
    info.ids_at = calib_at + 4 + g.n_calib * 8;
    return std::string();
}

std::string snapshot_parse(const uint8_t *bytes, size_t len, SnapshotInfo &info) {
    if (len >= 4 && (std::memcmp(bytes, "TVPI", 4) == 0 || std::memcmp(bytes, "TVIM", 4) == 0)) return parse_flat6(bytes, len, info);
    if (len < 23 || std::memcmp(bytes, "TV7\0", 4) != 0) return "not a TV7 image";
    if (bytes[4] != kVersion) return "unsupported TV7 revision " + std::to_string(bytes[4]);
    Geo g{};
    g.bits = bytes[5];
    g.kind = bytes[6];
    g.dim = int(get_u32(bytes + 7));
    if (g.bits < 2 || g.bits > 4) return "bit_width out of range";
    if (g.kind > 1) return "unknown index kind";
    if (g.dim <= 0 || g.dim % 8 != 0 || g.dim > 16384) return "dim out of range";
    if (get_u32(bytes + 19) != kMaxOps) return "op capacity differs from this build's";
    const size_t nl = g.n_levels();
    size_t off = 23 + (nl - 1) * 4 + nl * 4;
    if (len < off + 4) return "truncated superblock";
    g.n_calib = get_u32(bytes + off);
    if (g.n_calib != 0 && g.n_calib != size_t(g.dim)) return "calibration length is neither 0 nor dim";
    if (len < g.sb_len()) return "truncated superblock";
    if (get_u32(bytes + g.sb_len() - 4) != snapshot_crc32(bytes, g.sb_len() - 4)) return "superblock checksum mismatch";
    info.format = 7; info.kind = g.kind; info.dim = g.dim; info.bits = g.bits; info.n_calib = g.n_calib;
    info.boundaries_at = 23; info.centroids_at = 23 + (nl - 1) * 4;
    info.shift_at = off + 4; info.scale_at = off + 4 + g.n_calib * 4;

    if (len < g.sb_len() + 2 * g.hdr_len()) return "truncated header slots";
    const uint8_t *h = bytes + g.sb_len();
    if (get_u64(h) != 0) return "not a snapshot: generation is not 0 (a synced container needs the reference loader)";
    const uint64_t n = get_u64(h + 8);
    if (n >= (uint64_t(1) << 31)) return "row count out of range";
    const size_t n_tail = size_t(n % kBlock);
    const size_t row = g.row_bytes() + 4 + g.id_bytes(1);
    size_t at = 16 + n_tail * row;
    if (get_u32(h + at) != 0) return "not a snapshot: pending op groups present";
    at += 4;
    if (get_u32(h + at) != 0 || get_u32(h + at + 4) != 0 || get_u32(h + at + 8) != 0)
        return "not a snapshot: the commit names written units";
    DeltaDigest d(8);
    d.push(h, 8);
    if (get_u32(h + at + 12) != d.finish()) return "delta digest mismatch";
    at += 16;
    if (get_u32(h + at) != snapshot_crc32(h, at)) return "header checksum mismatch";
    if (len != g.unit_at(size_t(n) / kBlock)) return "image length does not match its row count";
    info.n = size_t(n);
    info.tail_at = g.sb_len() + 16;
    info.units_at = g.unit_at(0);
    info.unit_len = g.unit_len();
    info.row_bytes = g.row_bytes();
    return std::string();
}

// Rebuild sequential-blocked codes (ceil(n/32) blocks, padding lanes zero), scales and ids.
void snapshot_extract(const uint8_t *bytes, const SnapshotInfo &info, uint8_t *seq, float *scales, uint64_t *ids) {
    if (info.format == 6) {
        const size_t nb = (info.n + kBlock - 1) / kBlock;
        std::memcpy(seq, bytes + info.units_at, nb * info.row_bytes * kBlock);
        for (size_t i = 0; i < info.n; ++i) scales[i] = get_f32(bytes + info.tail_at + 4 * i);
        if (info.kind == 1 && ids) for (size_t i = 0; i < info.n; ++i) ids[i] = get_u64(bytes + info.ids_at + 8 * i);
        return;
    }
    const size_t G = info.row_bytes, n_blocks = info.n / kBlock, n_tail = info.n % kBlock;
    const bool has_ids = info.kind == 1;
    for (size_t b = 0; b < n_blocks; ++b) {
        const uint8_t *u = bytes + info.units_at + b * info.unit_len;
        std::memcpy(seq + b * G * kBlock, u, G * kBlock);
        for (size_t l = 0; l < kBlock; ++l) scales[b * kBlock + l] = get_f32(u + G * kBlock + 4 * l);
        if (has_ids && ids) for (size_t l = 0; l < kBlock; ++l) ids[b * kBlock + l] = get_u64(u + G * kBlock + 4 * kBlock + 8 * l);
    }
    if (n_tail) {
        uint8_t *blk = seq + n_blocks * G * kBlock;
        std::memset(blk, 0, G * kBlock);
        const uint8_t *p = bytes + info.tail_at;
        for (size_t k = 0; k < n_tail; ++k) {
            for (size_t gi = 0; gi < G; ++gi) blk[gi * kBlock + k] = p[gi];
            p += G;
            scales[n_blocks * kBlock + k] = get_f32(p); p += 4;
            if (has_ids) { if (ids) ids[n_blocks * kBlock + k] = get_u64(p); p += 8; }
        }
    }
}

}  // namespace tv
