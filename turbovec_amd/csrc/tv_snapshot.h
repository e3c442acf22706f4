// Snapshot images (turbovec/src/io_v7.rs): host-side composer and parser.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>

namespace tv {

struct SnapshotParts {
    int kind, dim, bits;              // kind 0: slot-addressed index, 1: id map (ids ride along)
    const float *boundaries, *centroids;
    size_t n_calib;                   // 0 or dim
    const float *shift, *scale;
    const uint8_t *seq;               // sequential-blocked codes, ceil(n/32) blocks (pack.rs:336-361)
    size_t n;
    const float *scales;
    const uint64_t *ids;              // kind 1 only
};

struct SnapshotInfo {
    int format = 7;                   // 7: TV7 snapshot image, 6: flat TVPI/TVIM container
    int kind = 0, dim = 0, bits = 0;
    size_t n_calib = 0, n = 0;
    size_t ids_at = 0;                // format 6 only
    size_t boundaries_at = 0, centroids_at = 0, shift_at = 0, scale_at = 0;
    size_t tail_at = 0, units_at = 0, unit_len = 0, row_bytes = 0;
};

uint32_t snapshot_crc32(const uint8_t *p, size_t n);
size_t snapshot_len(int format, int dim, int bits, int kind, size_t n_calib, size_t n);
void snapshot_compose(int format, const SnapshotParts &s, uint8_t *out);
std::string snapshot_parse(const uint8_t *bytes, size_t len, SnapshotInfo &info);
void snapshot_extract(const uint8_t *bytes, const SnapshotInfo &info, uint8_t *seq, float *scales, uint64_t *ids);

}  // namespace tv
