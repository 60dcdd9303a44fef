// CPU oracle (test infrastructure only, see oracle.h): int8 / fp8 quantized
// linears.  The reference has no implementation of these; the contract is the
// benchmark configuration (scale = absmax / 127 or absmax / 448,
// round-half-even, int32 or f32 accumulate, fused dequant).
#include "oracle.h"

#include <cmath>
#include <cstring>
#include <vector>

static inline int8_t quant_one(float x, float scale) {
    if (scale == 0.0f) return 0;
    float r = std::nearbyintf(x / scale);          // IEEE division, round-half-even
    if (r > 127.0f) r = 127.0f;
    if (r < -127.0f) r = -127.0f;
    return (int8_t)r;
}

extern "C" void orc_quantize_rows_i8(const float *x, size_t rows, size_t cols, int8_t *q,
                                     float *scale) {
    int nt = orc_get_threads();
#pragma omp parallel for schedule(static) num_threads(nt) if (rows > 1 && nt > 1)
    for (size_t r = 0; r < rows; ++r) {
        const float *row = x + r * cols;
        float amax = 0.0f;
        for (size_t c = 0; c < cols; ++c) amax = std::fmax(amax, std::fabs(row[c]));
        float s = amax / 127.0f;
        scale[r] = s;
        for (size_t c = 0; c < cols; ++c) q[r * cols + c] = quant_one(row[c], s);
    }
}

extern "C" void orc_quantize_cols_i8(const float *w, size_t k, size_t n, int8_t *q, float *scale) {
    std::vector<float> amax(n, 0.0f);
    for (size_t p = 0; p < k; ++p)
        for (size_t j = 0; j < n; ++j) amax[j] = std::fmax(amax[j], std::fabs(w[p * n + j]));
    for (size_t j = 0; j < n; ++j) scale[j] = amax[j] / 127.0f;
    int nt = orc_get_threads();
#pragma omp parallel for schedule(static) num_threads(nt) if (k > 1 && nt > 1)
    for (size_t p = 0; p < k; ++p)
        for (size_t j = 0; j < n; ++j) q[p * n + j] = quant_one(w[p * n + j], scale[j]);
}

extern "C" void orc_gemm_i8_i32(const int8_t *a, const int8_t *b, const int32_t *c_in,
                                int32_t *acc, size_t m, size_t n, size_t k) {
    int nt = orc_get_threads();
#pragma omp parallel for schedule(static) num_threads(nt) if (m > 1 && nt > 1)
    for (size_t i = 0; i < m; ++i) {
        int32_t *row = acc + i * n;
        for (size_t j = 0; j < n; ++j) row[j] = c_in ? c_in[i * n + j] : 0;
        for (size_t p = 0; p < k; ++p) {
            int32_t av = (int32_t)a[i * k + p];
            const int8_t *b_row = b + p * n;
            // wrapping arithmetic like the hardware accumulator
            for (size_t j = 0; j < n; ++j)
                row[j] = (int32_t)((uint32_t)row[j] + (uint32_t)(av * (int32_t)b_row[j]));
        }
    }
}

extern "C" void orc_dequant_i32(const int32_t *acc, const float *sx, const float *sw,
                                const float *bias, float *out, size_t m, size_t n) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) {
            float s = sx[i] * sw[j];
            float v = (float)acc[i * n + j] * s;
            if (bias) v = v + bias[j];
            out[i * n + j] = v;
        }
}

extern "C" void orc_linear_w8a8(const float *x, const int8_t *wq, const float *sw,
                                const float *bias, int32_t *acc_out, float *out, size_t m,
                                size_t n, size_t k) {
    std::vector<int8_t> xq(m * k);
    std::vector<float> sx(m);
    orc_quantize_rows_i8(x, m, k, xq.data(), sx.data());
    std::vector<int32_t> tmp;
    int32_t *acc = acc_out;
    if (!acc) {
        tmp.resize(m * n);
        acc = tmp.data();
    }
    orc_gemm_i8_i32(xq.data(), wq, nullptr, acc, m, n, k);
    orc_dequant_i32(acc, sx.data(), sw, bias, out, m, n);
}

extern "C" void orc_linear_w8a16(const uint16_t *a_bf16, const int8_t *wq, const float *sw,
                                 float *out_f32, size_t m, size_t n, size_t k) {
    int nt = orc_get_threads();
    // columns are split over threads; each output keeps one accumulator, k ascending
#pragma omp parallel num_threads(nt) if (nt > 1)
    {
        std::vector<float> accv;
#pragma omp for schedule(static)
        for (size_t jb = 0; jb < (n + 255) / 256; ++jb) {
            size_t j0 = jb * 256, j1 = j0 + 256 < n ? j0 + 256 : n;
            accv.assign((j1 - j0) * m, 0.0f);
            for (size_t p = 0; p < k; ++p) {
                const int8_t *w_row = wq + p * n;
                for (size_t i = 0; i < m; ++i) {
                    float av = orc_bf16_to_f32(a_bf16[i * k + p]);
                    float *acc = accv.data() + i * (j1 - j0);
                    for (size_t j = j0; j < j1; ++j)
                        acc[j - j0] = std::fmaf(av, (float)w_row[j], acc[j - j0]);
                }
            }
            for (size_t i = 0; i < m; ++i)
                for (size_t j = j0; j < j1; ++j)
                    out_f32[i * n + j] = accv[i * (j1 - j0) + (j - j0)] * sw[j];
        }
    }
}

extern "C" float orc_quantize_tensor_e4m3(const float *x, size_t n, uint8_t *q) {
    float amax = 0.0f;
    for (size_t i = 0; i < n; ++i) amax = std::fmax(amax, std::fabs(x[i]));
    float s = amax / 448.0f;
    for (size_t i = 0; i < n; ++i) q[i] = s == 0.0f ? 0 : orc_f32_to_e4m3(x[i] / s);
    return s;
}

extern "C" void orc_quantize_rows_e4m3(const float *x, size_t rows, size_t cols, uint8_t *q, float *scale) {
    int nt = orc_get_threads();
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (size_t r = 0; r < rows; ++r) {
        float amax = 0.0f;
        for (size_t c = 0; c < cols; ++c) amax = std::fmax(amax, std::fabs(x[r * cols + c]));
        float s = amax / 448.0f;
        scale[r] = s;
        for (size_t c = 0; c < cols; ++c) q[r * cols + c] = s == 0.0f ? 0 : orc_f32_to_e4m3(x[r * cols + c] / s);
    }
}

extern "C" void orc_quantize_cols_e4m3(const float *w, size_t k, size_t n, uint8_t *q, float *scale) {
    int nt = orc_get_threads();
#pragma omp parallel for num_threads(nt) schedule(static) if (nt > 1)
    for (size_t c = 0; c < n; ++c) {
        float amax = 0.0f;
        for (size_t r = 0; r < k; ++r) amax = std::fmax(amax, std::fabs(w[r * n + c]));
        float s = amax / 448.0f;
        scale[c] = s;
        for (size_t r = 0; r < k; ++r) q[r * n + c] = s == 0.0f ? 0 : orc_f32_to_e4m3(w[r * n + c] / s);
    }
}

extern "C" void orc_linear_e4m3_rows(const uint8_t *a, const uint8_t *b, const float *sa, const float *sb,
                                     const float *bias, float *out, size_t m, size_t n, size_t k) {
    float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = orc_e4m3_to_f32((uint8_t)i);
    int nt = orc_get_threads();
#pragma omp parallel num_threads(nt) if (nt > 1)
    {
        std::vector<double> acc(n);
#pragma omp for schedule(static)
        for (size_t i = 0; i < m; ++i) {
            std::fill(acc.begin(), acc.end(), 0.0);
            for (size_t p = 0; p < k; ++p) {
                double av = (double)lut[a[i * k + p]];
                const uint8_t *b_row = b + p * n;
                for (size_t j = 0; j < n; ++j) acc[j] += av * (double)lut[b_row[j]];
            }
            for (size_t j = 0; j < n; ++j) {
                float v = (float)acc[j] * (sa[i] * sb[j]);
                out[i * n + j] = bias ? v + bias[j] : v;
            }
        }
    }
}

extern "C" void orc_gemm_e4m3(const uint8_t *a, const uint8_t *b, float sa, float sb, float *out,
                              size_t m, size_t n, size_t k) {
    float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = orc_e4m3_to_f32((uint8_t)i);
    float s = sa * sb;
    int nt = orc_get_threads();
#pragma omp parallel num_threads(nt) if (nt > 1)
    {
        std::vector<double> acc(n);
#pragma omp for schedule(static)
        for (size_t i = 0; i < m; ++i) {
            std::fill(acc.begin(), acc.end(), 0.0);
            for (size_t p = 0; p < k; ++p) {
                double av = (double)lut[a[i * k + p]];
                const uint8_t *b_row = b + p * n;
                for (size_t j = 0; j < n; ++j) acc[j] += av * (double)lut[b_row[j]];
            }
            for (size_t j = 0; j < n; ++j) out[i * n + j] = (float)acc[j] * s;
        }
    }
}
