#include "host_tables.h"

#include <algorithm>
#include <cstring>

#include <array>
#include <cfloat>
#include <cmath>
#include <functional>
#include <map>
#include <mutex>
#include <utility>

namespace tv {
namespace {

// ChaCha with 8 rounds as rand_chacha 0.3.1 drives it for ChaCha8Rng: 64-bit
// block counter in state words 12-13, stream id zero, output consumed as a
// flat sequence of little-endian u32 words (turbovec/Cargo.toml:49).
class ChaCha8Words {
public:
    explicit ChaCha8Words(const std::array<uint8_t, 32> &seed) {
        for (int i = 0; i < 8; ++i) {
            key_[i] = uint32_t(seed[4 * i]) | uint32_t(seed[4 * i + 1]) << 8 |
                      uint32_t(seed[4 * i + 2]) << 16 | uint32_t(seed[4 * i + 3]) << 24;
        }
    }
    uint32_t word() {
        if (pos_ == 16) { refill(); }
        return block_[pos_++];
    }
    // rand_core's BlockRng::next_u64 reads the low half first.  Word reads and
    // pair reads share one flat stream, so buffering per 16-word block gives the
    // same sequence as the crate's 64-word buffer.
    uint64_t pair() {
        uint64_t lo = word();
        uint64_t hi = word();
        return hi << 32 | lo;
    }

private:
    static uint32_t rol(uint32_t v, int s) { return v << s | v >> (32 - s); }
    static void quarter(uint32_t *s, int a, int b, int c, int d) {
        s[a] += s[b]; s[d] = rol(s[d] ^ s[a], 16);
        s[c] += s[d]; s[b] = rol(s[b] ^ s[c], 12);
        s[a] += s[b]; s[d] = rol(s[d] ^ s[a], 8);
        s[c] += s[d]; s[b] = rol(s[b] ^ s[c], 7);
    }
    void refill() {
        uint32_t init[16] = {0x61707865u, 0x3320646eu, 0x79622d32u, 0x6b206574u};
        for (int i = 0; i < 8; ++i) init[4 + i] = key_[i];
        init[12] = uint32_t(counter_);
        init[13] = uint32_t(counter_ >> 32);
        init[14] = init[15] = 0;
        uint32_t s[16];
        for (int i = 0; i < 16; ++i) s[i] = init[i];
        for (int round = 0; round < 8; round += 2) {
            quarter(s, 0, 4, 8, 12); quarter(s, 1, 5, 9, 13);
            quarter(s, 2, 6, 10, 14); quarter(s, 3, 7, 11, 15);
            quarter(s, 0, 5, 10, 15); quarter(s, 1, 6, 11, 12);
            quarter(s, 2, 7, 8, 13); quarter(s, 3, 4, 9, 14);
        }
        for (int i = 0; i < 16; ++i) block_[i] = s[i] + init[i];
        ++counter_;
        pos_ = 0;
    }
    uint32_t key_[8];
    uint32_t block_[16];
    uint64_t counter_ = 0;
    int pos_ = 16;
};

// turbovec/src/rotation.rs:82-85
constexpr std::array<uint8_t, 32> kRotationSeed = {
    164, 143, 161, 123, 88, 50, 61, 10, 234, 184, 161, 204, 105, 1, 20, 184,
    43, 140, 200, 117, 24, 180, 247, 84, 141, 68, 110, 161, 228, 223, 32, 242};

// Regularised incomplete beta I_x(a, a) as statrs 0.17.1 evaluates Beta::cdf
// (turbovec/Cargo.toml:67): continued fraction by the modified Lentz method.
double incomplete_beta_sym(double shape, double x) {
    if (x <= 0.0) return 0.0;
    if (x >= 1.0) return 1.0;
    double a = shape, b = shape;
    const double front = std::exp(std::lgamma(a + b) - std::lgamma(a) - std::lgamma(b) +
                                  a * std::log(x) + b * std::log(1.0 - x));
    const bool mirrored = x >= (a + 1.0) / (a + b + 2.0);
    if (mirrored) { x = 1.0 - x; }
    const double tiny = DBL_MIN / 1.1102230246251565e-16;
    auto guard = [tiny](double v) { return std::fabs(v) < tiny ? tiny : v; };
    double c = 1.0;
    double d = 1.0 / guard(1.0 - (a + b) * x / (a + 1.0));
    double frac = d;
    for (int step = 1; step <= 140; ++step) {
        const double m = step, two_m = 2.0 * m;
        double term = m * (b - m) * x / ((a - 1.0 + two_m) * (a + two_m));
        d = 1.0 / guard(1.0 + term * d);
        c = guard(1.0 + term / c);
        frac *= d * c;
        term = -(a + m) * (a + b + m) * x / ((a + two_m) * (a + 1.0 + two_m));
        d = 1.0 / guard(1.0 + term * d);
        c = guard(1.0 + term / c);
        const double delta = d * c;
        frac *= delta;
        if (std::fabs(delta - 1.0) <= 1.1102230246251565e-16) break;
    }
    const double tail = front * frac / a;
    return mirrored ? 1.0 - tail : tail;
}

double beta_density_sym(double shape, double x) {
    if (x < 0.0 || x > 1.0) return 0.0;
    if (shape > 80.0) {
        const double lognorm = std::lgamma(2.0 * shape) - 2.0 * std::lgamma(shape);
        const double lx = x == 0.0 ? -INFINITY : (shape - 1.0) * std::log(x);
        const double l1x = x == 1.0 ? -INFINITY : (shape - 1.0) * std::log(1.0 - x);
        return std::exp(lognorm + lx + l1x);
    }
    const double norm = std::tgamma(2.0 * shape) / (std::tgamma(shape) * std::tgamma(shape));
    return norm * std::pow(x, shape - 1.0) * std::pow(1.0 - x, shape - 1.0);
}

// turbovec/src/codebook.rs:214-249
struct Simpson {
    std::function<double(double)> f;
    double run(double lo, double hi, double tol, int depth) const {
        const double fl = f(lo), fh = f(hi), fm = f((lo + hi) / 2.0);
        return refine(lo, hi, fl, fh, fm, (hi - lo) / 6.0 * (fl + 4.0 * fm + fh), tol, depth);
    }
    double refine(double lo, double hi, double fl, double fh, double fm, double whole, double tol,
                  int depth) const {
        const double mid = (lo + hi) / 2.0;
        const double q1 = (lo + mid) / 2.0, q3 = (mid + hi) / 2.0;
        const double f1 = f(q1), f3 = f(q3);
        const double left = (mid - lo) / 6.0 * (fl + 4.0 * f1 + fm);
        const double right = (hi - mid) / 6.0 * (fm + 4.0 * f3 + fh);
        const double both = left + right;
        if (depth == 0 || std::fabs(both - whole) < 15.0 * tol) return both + (both - whole) / 15.0;
        return refine(lo, mid, fl, fm, f1, left, tol / 2.0, depth - 1) +
               refine(mid, hi, fm, fh, f3, right, tol / 2.0, depth - 1);
    }
};

}  // namespace

RotationTables make_rotation_tables(int dim) {
    RotationTables t;
    t.dim = dim;
    t.block = dim & -dim;
    t.inv_sqrt_block = 1.0f / std::sqrt(float(t.block));
    t.signs.resize(size_t(2) * dim);
    t.perms.resize(size_t(2) * dim);
    ChaCha8Words rng(kRotationSeed);
    for (int round = 0; round < 2; ++round) {
        float *sg = t.signs.data() + size_t(round) * dim;
        uint32_t *pm = t.perms.data() + size_t(round) * dim;
        for (int i = 0; i < dim; ++i) sg[i] = (rng.word() & 1u) ? -1.0f : 1.0f;
        for (int i = 0; i < dim; ++i) pm[i] = uint32_t(i);
        for (int i = dim - 1; i > 0; --i) std::swap(pm[i], pm[rng.pair() % (uint64_t(i) + 1)]);
    }
    return t;
}

Codebook make_codebook(int bits, int dim) {
    static std::mutex mu;
    static std::map<std::pair<int, int>, Codebook> memo;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto hit = memo.find({bits, dim});
        if (hit != memo.end()) return hit->second;
    }
    const double shape = (double(dim) - 1.0) / 2.0;
    const int levels = 1 << bits;
    std::vector<double> cen(levels), next(levels), edge(levels + 1);
    const double sigma = std::sqrt(2.0 * shape / ((2.0 * shape + 1.0) * 4.0 * shape));
    for (int i = 0; i < levels; ++i) cen[i] = -3.0 * sigma + 2.0 * (3.0 * sigma) * double(i) / (double(levels) - 1.0);
    Simpson mean_integral{[shape](double x) { return x * beta_density_sym(shape, (x + 1.0) / 2.0) / 2.0; }};
    for (int iter = 0; iter < 200; ++iter) {
        edge[0] = -1.0;
        edge[levels] = 1.0;
        for (int i = 1; i < levels; ++i) edge[i] = (cen[i - 1] + cen[i]) / 2.0;
        double moved = 0.0;
        for (int i = 0; i < levels; ++i) {
            const double mass = incomplete_beta_sym(shape, (edge[i + 1] + 1.0) / 2.0) -
                                incomplete_beta_sym(shape, (edge[i] + 1.0) / 2.0);
            next[i] = mass < 1e-15 ? cen[i] : mean_integral.run(edge[i], edge[i + 1], 1e-14, 50) / mass;
            moved = std::fmax(moved, std::fabs(next[i] - cen[i]));
        }
        cen = next;
        if (moved < 1e-12) break;
    }
    Codebook cb;
    cb.centroids.resize(levels);
    cb.boundaries.resize(levels - 1);
    for (int i = 0; i < levels; ++i) cb.centroids[i] = float(cen[i]);
    // Midpoints are taken between the already-rounded f32 centroids (codebook.rs:161-166).
    for (int i = 0; i + 1 < levels; ++i) cb.boundaries[i] = (cb.centroids[i] + cb.centroids[i + 1]) * 0.5f;
    std::lock_guard<std::mutex> lock(mu);
    memo[{bits, dim}] = cb;
    return cb;
}

void fit_tqplus(const float *rotated, size_t n, int dim, const std::vector<float> &centroids,
                float *shift, float *scale) {
    float c_outer = 0.0f;
    for (float c : centroids) c_outer = std::fmax(c_outer, std::fabs(c));
    const double shape = (double(dim) - 1.0) / 2.0;
    const double p_hi = incomplete_beta_sym(shape, (double(c_outer) + 1.0) / 2.0);   // encode.rs:364-369
    const double p_lo = 1.0 - p_hi;
    const float qc_lo = -c_outer, qc_span = c_outer - qc_lo;
    size_t lo_idx = size_t(double(n) * p_lo);
    size_t hi_idx = size_t(double(n) * p_hi);
    if (hi_idx > n - 1) hi_idx = n - 1;
    if (hi_idx < lo_idx + 1) hi_idx = lo_idx + 1;
    // total order of encode.rs:183-186: sign-magnitude bits mapped to unsigned keys
    auto key = [](float x) { uint32_t b; std::memcpy(&b, &x, 4); return b ^ (uint32_t(int32_t(b) >> 31) | 0x80000000u); };
    auto unkey = [](uint32_t k) { const uint32_t b = k ^ ((k & 0x80000000u) ? 0x80000000u : 0xFFFFFFFFu); float x; std::memcpy(&x, &b, 4); return x; };
    std::vector<uint32_t> col(n);
    for (int d = 0; d < dim; ++d) {
        shift[d] = 0.0f;
        scale[d] = 1.0f;
        if (n < 2 || hi_idx >= n) continue;
        for (size_t i = 0; i < n; ++i) col[i] = key(rotated[i * size_t(dim) + d]);
        std::nth_element(col.begin(), col.begin() + lo_idx, col.end());
        const float qe_lo = unkey(col[lo_idx]);
        std::nth_element(col.begin() + lo_idx + 1, col.begin() + hi_idx, col.end());   // hi_idx > lo_idx
        const float qe_hi = unkey(col[hi_idx]);
        const float qe_span = qe_hi - qe_lo;
        if (qe_span > 1e-6f) {
            scale[d] = qc_span / qe_span;
            shift[d] = qc_lo / scale[d] - qe_lo;
        }
    }
}

}  // namespace tv
