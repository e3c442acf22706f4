// Host-side derivation of the tables the search kernels read: the rotation's
// sign/permutation rounds and the Lloyd-Max centroids.  Pure functions of
// (dim, bits); computed once per index at creation.
#pragma once
#include <cstdint>
#include <vector>

namespace tv {

struct RotationTables {
    int dim = 0;
    int block = 0;             // largest power-of-two divisor of dim
    float inv_sqrt_block = 0;  // 1 / sqrt(block), rounded once in f32
    std::vector<float> signs;     // round 0 then round 1, dim each
    std::vector<uint32_t> perms;  // round 0 then round 1, dim each
};

// turbovec/src/rotation.rs:141-187 (Rotation::new) and :990-997 (fisher_yates).
RotationTables make_rotation_tables(int dim);

struct Codebook {
    std::vector<float> boundaries;  // 2^bits - 1
    std::vector<float> centroids;   // 2^bits
};

// turbovec/src/codebook.rs:69-167 (lloyd_max, 200 iterations, tol 1e-12).
Codebook make_codebook(int bits, int dim);

// turbovec/src/encode.rs:737-857 (compute_tqplus_calibration) given the rotated unit rows
// (n * dim floats, row-major): per coordinate, the order statistics at the tail
// probabilities of the outer centroid under Beta((dim-1)/2, (dim-1)/2) are mapped onto
// +-outer centroid.  shift and scale receive dim floats each.
void fit_tqplus(const float *rotated, size_t n, int dim, const std::vector<float> &centroids,
                float *shift, float *scale);

}  // namespace tv
