// CPU oracle (test infrastructure only, see oracle.h): rng, tolerance judge,
// number formats, f32 GEMM / linear, RMSNorm, RoPE, elementwise, pool classes.
// Built with -ffp-contract=off: a fused multiply-add appears only where the
// reference calls mul_add, written here as an explicit fma.
#include "oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <vector>

static int g_threads = 1;

extern "C" int orc_set_threads(int n) {
    g_threads = n < 1 ? 1 : n;
    return g_threads;
}
extern "C" int orc_get_threads(void) { return g_threads; }

// ------------------------------------------------------------------- rng
// crates/tensor-core/src/rng.rs:62-105
extern "C" uint64_t orc_rng_init(uint64_t seed) {
    return seed == 0 ? 0x9E3779B97F4A7C15ull : seed;
}
extern "C" uint64_t orc_rng_next_u64(uint64_t *state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return x * 0x2545F4914F6CDD1Dull;
}
extern "C" float orc_rng_next_unit_f32(uint64_t *state) {
    uint32_t bits = (uint32_t)(orc_rng_next_u64(state) >> 40);
    return (float)bits / (float)(1u << 24);
}
extern "C" float orc_rng_next_f32(uint64_t *state) {
    float unit = orc_rng_next_unit_f32(state);
    return unit * 2.0f - 1.0f;
}
extern "C" double orc_rng_next_unit_f64(uint64_t *state) {
    uint64_t bits = orc_rng_next_u64(state) >> 11;
    return (double)bits / (double)(1ull << 53);
}
// crates/tensor-core/src/rng.rs:231-255
extern "C" void orc_randn_f32(uint64_t *state, float *out, size_t n, float std) {
    const double tau = 6.283185307179586476925286766559;
    size_t i = 0;
    while (i < n) {
        double u1 = 1.0 - orc_rng_next_unit_f64(state);
        double u2 = orc_rng_next_unit_f64(state);
        double r = std::sqrt(-2.0 * std::log(u1));
        double theta = tau * u2;
        out[i++] = (float)(r * std::cos(theta)) * std;
        if (i == n) break;
        out[i++] = (float)(r * std::sin(theta)) * std;
    }
}
extern "C" void orc_rand_unit_f32(uint64_t *state, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_rng_next_unit_f32(state);
}
extern "C" void orc_rand_pm1_f32(uint64_t *state, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_rng_next_f32(state);
}
// crates/tensor-core/src/rng.rs:283-312
static uint64_t draw_below(uint64_t *state, uint64_t range) {
    uint64_t zone = range * (UINT64_MAX / range);
    for (;;) {
        uint64_t x = orc_rng_next_u64(state);
        if (x < zone) return x % range;
    }
}
extern "C" int orc_randint(uint64_t *state, int32_t low, int32_t high, int32_t *out, size_t n) {
    if (low >= high) return -1;
    uint64_t range = (uint64_t)((int64_t)high - (int64_t)low);
    for (size_t i = 0; i < n; ++i) out[i] = (int32_t)((int64_t)low + (int64_t)draw_below(state, range));
    return 0;
}
extern "C" void orc_permutation_u32(uint64_t *state, uint32_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = (uint32_t)i;
    for (size_t i = n; i > 1; --i) {
        size_t j = (size_t)draw_below(state, (uint64_t)i);
        std::swap(out[i - 1], out[j]);
    }
}
// crates/backend-cpu/tests/paged_kv_backend_parity.rs:21-31
extern "C" void orc_test_data_f32(float *out, size_t n, uint64_t seed) {
    uint64_t s = (seed * 0x9E3779B97F4A7C15ull) | 1ull;
    for (size_t i = 0; i < n; ++i) {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        out[i] = ((float)(s >> 40) / (float)(1ull << 24)) * 2.0f - 1.0f;
    }
}

// ------------------------------------------------------------- tolerance
// crates/tensor-core/src/tolerance.rs:15-37
extern "C" int orc_composite_close_f32(float actual, float reference) {
    double a = (double)actual, b = (double)reference;
    double diff = std::fabs(a - b);
    double scale = std::fmax(std::fmax(std::fabs(a), std::fabs(b)), 1e-12);
    double rel = diff / scale;
    return (rel < 1e-3 || diff < 1e-5) ? 1 : 0;
}

static double percentile(const std::vector<double> &sorted, double p) {
    if (sorted.empty()) return 0.0;
    size_t idx = (size_t)std::llround(((double)sorted.size() - 1.0) * p);
    return sorted[std::min(idx, sorted.size() - 1)];
}
static double max_nonfinite_aware(const std::vector<double> &v) {
    double acc = 0.0;
    for (double x : v) {
        if (!std::isfinite(x)) return INFINITY;
        acc = std::max(acc, x);
    }
    return acc;
}
// crates/backend-cpu/src/parity.rs:138-245
extern "C" void orc_compare_f32(const float *actual, const float *reference, size_t n,
                                orc_compare_report *out) {
    std::vector<double> abs_diffs(n), rel_errs(n);
    uint64_t fail = 0, bits = 0;
    double max_fail = 0.0;
    for (size_t i = 0; i < n; ++i) {
        double x = (double)actual[i], y = (double)reference[i];
        double diff = std::fabs(x - y);
        double scale = std::fmax(std::fmax(std::fabs(x), std::fabs(y)), 1e-12);
        double rel = diff / scale;
        bool pass = rel < 1e-3 || diff < 1e-5;
        if (!pass) {
            ++fail;
            max_fail = std::isfinite(diff) ? std::max(max_fail, diff) : INFINITY;
        }
        abs_diffs[i] = diff;
        rel_errs[i] = rel;
        uint32_t ba, bb;
        std::memcpy(&ba, &actual[i], 4);
        std::memcpy(&bb, &reference[i], 4);
        if (ba != bb) ++bits;
    }
    out->total = n;
    out->fail_count = fail;
    out->max_abs_diff = max_nonfinite_aware(abs_diffs);
    out->max_rel_err = max_nonfinite_aware(rel_errs);
    double sa = 0.0, sr = 0.0;
    for (size_t i = 0; i < n; ++i) {
        sa += abs_diffs[i];
        sr += rel_errs[i];
    }
    out->mean_abs_diff = n ? sa / (double)n : 0.0;
    out->mean_rel_err = n ? sr / (double)n : 0.0;
    std::vector<double> sorted = abs_diffs;
    std::sort(sorted.begin(), sorted.end(), [](double a, double b) { return a < b; });
    out->p50_abs_diff = percentile(sorted, 0.50);
    out->p99_abs_diff = percentile(sorted, 0.99);
    out->p999_abs_diff = percentile(sorted, 0.999);
    out->max_fail_abs_diff = max_fail;
    out->bit_mismatch = bits;
}

// --------------------------------------------------------- number formats
extern "C" uint16_t orc_f32_to_bf16(float v) {
    uint32_t u;
    std::memcpy(&u, &v, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    uint32_t round = 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + round) >> 16);
}
extern "C" float orc_bf16_to_f32(uint16_t v) {
    uint32_t u = (uint32_t)v << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
extern "C" void orc_f32_to_bf16_n(const float *in, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}
extern "C" void orc_bf16_to_f32_n(const uint16_t *in, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]);
}

extern "C" float orc_e4m3_to_f32(uint8_t v) {
    int sign = v >> 7;
    int exp = (v >> 3) & 0xf;
    int man = v & 7;
    float mag;
    if (exp == 0xf && man == 7) return NAN;
    if (exp == 0) mag = std::ldexp((float)man, -9);                // subnormal: man * 2^-6 / 8
    else mag = std::ldexp(1.0f + (float)man / 8.0f, exp - 7);
    return sign ? -mag : mag;
}
extern "C" uint8_t orc_f32_to_e4m3(float v) {
    if (std::isnan(v)) return 0x7f;
    uint8_t sign = std::signbit(v) ? 0x80 : 0x00;
    double a = std::fabs((double)v);
    if (a >= 464.0) return sign | 0x7e;         // at or above the 448|480 midpoint: saturate
    if (a == 0.0) return sign;
    int e;
    (void)std::frexp(a, &e);                    // a = f * 2^e, f in [0.5, 1)
    int exp_unb = e - 1;                        // a in [2^exp_unb, 2^(exp_unb+1))
    if (exp_unb < -6) exp_unb = -6;             // subnormal range shares the 2^-6 spacing / 8
    double step = std::ldexp(1.0, exp_unb - 3); // spacing of representable values in this binade
    double q = std::nearbyint(a / step);        // round-half-even (default rounding mode)
    double r = q * step;
    if (r > 448.0) r = 448.0;
    // re-derive the fields from the rounded magnitude (rounding may carry into the next binade)
    if (r == 0.0) return sign;
    int e2;
    double f2 = std::frexp(r, &e2);
    int eu = e2 - 1;
    uint8_t code;
    if (eu < -6) {
        code = (uint8_t)std::lround(std::ldexp(r, 9));             // subnormal mantissa
    } else {
        int man = (int)std::lround((f2 * 2.0 - 1.0) * 8.0);
        code = (uint8_t)(((eu + 7) << 3) | man);
    }
    return sign | code;
}
extern "C" void orc_f32_to_e4m3_n(const float *in, uint8_t *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_e4m3(in[i]);
}
extern "C" void orc_e4m3_to_f32_n(const uint8_t *in, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_to_f32(in[i]);
}

// --------------------------------------------------------- f32 GEMM/linear
// crates/backend-cpu/src/parity.rs:340-361 / gemm.rs:230-257.  The loop nest
// is i-k-j like the reference; every c[i][j] still sees k ascending with one
// accumulator, so splitting rows over threads changes no result.
extern "C" void orc_gemm_f32(const float *a, const float *b, float *c, size_t m, size_t n,
                             size_t k) {
#pragma omp parallel for schedule(static) num_threads(g_threads) if (m > 1 && g_threads > 1)
    for (size_t i = 0; i < m; ++i) {
        float *c_row = c + i * n;
        for (size_t j = 0; j < n; ++j) c_row[j] = 0.0f;
        const float *a_row = a + i * k;
        for (size_t p = 0; p < k; ++p) {
            float a_ip = a_row[p];
            const float *b_row = b + p * n;
            for (size_t j = 0; j < n; ++j) c_row[j] = std::fmaf(a_ip, b_row[j], c_row[j]);
        }
    }
}
// crates/backend-cpu/src/ops.rs:514-643: bias added after the product, then
// the activation (none | relu = max(0, x)).
extern "C" void orc_linear_f32(const float *a, const float *w, const float *bias, float *y,
                               size_t m, size_t n, size_t k, int act) {
    orc_gemm_f32(a, w, y, m, n, k);
    for (size_t i = 0; i < m; ++i) {
        float *row = y + i * n;
        for (size_t j = 0; j < n; ++j) {
            float v = row[j];
            if (bias) v = v + bias[j];
            if (act == 1) v = v > 0.0f ? v : (std::isnan(v) ? v : 0.0f);
            row[j] = v;
        }
    }
}

// ----------------------------------------------------------------- RMSNorm
// crates/backend-cpu/src/rmsnorm.rs:90-228
static void rmsnorm_row(const float *row, const float *w, float eps, float inv_n, size_t hidden,
                        float *out) {
    double acc = 0.0;
    for (size_t i = 0; i < hidden; ++i) {
        double v = (double)row[i];
        acc = std::fma(v, v, acc);
    }
    float rstd = (float)(1.0 / std::sqrt(std::fma(acc, (double)inv_n, (double)eps)));
    if (w) {
        for (size_t i = 0; i < hidden; ++i) {
            float t = row[i] * rstd;
            out[i] = t * w[i];
        }
    } else {
        for (size_t i = 0; i < hidden; ++i) out[i] = row[i] * rstd;
    }
}
extern "C" int orc_rmsnorm_f32(const float *x, const float *w, size_t w_len, float eps,
                               size_t rows, size_t hidden, size_t x_len, float *out) {
    if (!std::isfinite(eps) || eps < 0.0f) return -1;
    if (hidden != 0 && rows > SIZE_MAX / hidden) return -2;
    if (rows * hidden != x_len) return -2;
    if (w && w_len != hidden) return -3;
    if (rows == 0 || hidden == 0) return 0;
    float inv_n = 1.0f / (float)hidden;
#pragma omp parallel for schedule(static) num_threads(g_threads) if (rows > 1 && g_threads > 1)
    for (size_t r = 0; r < rows; ++r) rmsnorm_row(x + r * hidden, w, eps, inv_n, hidden, out + r * hidden);
    return 0;
}

// -------------------------------------------------------------------- RoPE
extern "C" void orc_rope_f32(const float *x, const int32_t *positions, size_t rows, size_t heads,
                             size_t head_dim, double theta, float *out) {
    size_t half = head_dim / 2;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t i = 0; i < half; ++i) {
            double inv_freq = std::pow(theta, -2.0 * (double)i / (double)head_dim);
            double angle = (double)positions[r] * inv_freq;
            float c = (float)std::cos(angle), s = (float)std::sin(angle);
            for (size_t h = 0; h < heads; ++h) {
                size_t base = (r * heads + h) * head_dim;
                float xi = x[base + i], xj = x[base + i + half];
                float a = xi * c, b = xj * s, d = xj * c, e = xi * s;
                out[base + i] = a - b;
                out[base + i + half] = d + e;
            }
        }
    }
}

// ------------------------------------------------------------ elementwise
// crates/tensor-core/src/scalar_op.rs:666-673 sigmoid_stable, :355 Silu
extern "C" float orc_silu_f32(float x) {
    float s;
    if (x >= 0.0f) {
        s = 1.0f / (1.0f + std::exp(-x));
    } else {
        float e = std::exp(x);
        s = e / (1.0f + e);
    }
    return x * s;
}
extern "C" void orc_silu_mul_f32(const float *gate, const float *up, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_silu_f32(gate[i]) * up[i];
}
extern "C" void orc_add_f32(const float *a, const float *b, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}
// crates/autodiff/src/generate/mod.rs:333-343; NaN rule crates/backend-rocm/src/ops.rs:991-995
extern "C" void orc_argmax_rows_f32(const float *x, size_t rows, size_t cols, int32_t *out) {
    for (size_t r = 0; r < rows; ++r) {
        const float *row = x + r * cols;
        size_t best = 0;
        bool have = false;
        float best_val = 0.0f;
        for (size_t i = 0; i < cols; ++i) {
            float v = row[i];
            if (std::isnan(v)) continue;
            if (!have || v > best_val) {
                have = true;
                best_val = v;
                best = i;
            }
        }
        out[r] = (int32_t)best;
    }
}

// ------------------------------------------------------------ memory pool
// crates/tensor-core/src/pool_core.rs:157-209, default config :102-112
extern "C" uint64_t orc_size_class_for(uint64_t bytes) {
    const uint64_t small_max = 1024ull * 1024, granule = 2ull * 1024 * 1024,
                   huge_min = 64ull * 1024 * 1024;
    if (bytes == 0) return 0;
    if (bytes >= huge_min) return bytes;
    if (bytes > small_max) {
        if (bytes > UINT64_MAX - (granule - 1)) return UINT64_MAX;
        return (bytes + granule - 1) / granule * granule;
    }
    if (bytes <= 255) return 256;
    int octave = 63 - __builtin_clzll(bytes);
    uint64_t base = 1ull << octave;
    uint64_t step = base / 4;
    for (uint64_t mult = 4; mult <= 7; ++mult) {
        uint64_t cls = base + step * (mult - 4);
        if (cls >= bytes) return cls;
    }
    return base * 2;
}
