/* CPU oracle, C restatement (TEST INFRASTRUCTURE ONLY; never linked into the product).
 *
 * An independent second statement of the E8P codebook, decoder, two-stage Q4
 * weights, A8 quantiser and the int32 contraction + fp32 rescale, written with
 * integer loops only (no BLAS, no fp64 trick), so that it cross-checks the
 * numpy oracle in reference.py.  Reference lines followed:
 *   basis        python/orinfer_build/quantization/e8p.py:15-25
 *   decode       python/orinfer_build/quantization/vq.py:17,34-43
 *   q4 weights   python/orinfer_build/quantization/e8p_q4.py:61-67
 *   a8           python/orinfer_build/quantization/reference_math.py:6-20
 *   rescale      kernels/cuda/model/integer_core.py:19-22
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static const int SIGN_BITS[8] = {0, 4, 1, 5, 2, 6, 3, 7};

/* Next 5-subset of {0..7} in lexicographic order; returns 0 when exhausted. */
static int next_subset(int *c) {
    int i = 4;
    while (i >= 0 && c[i] == 8 - 5 + i) --i;
    if (i < 0) return 0;
    ++c[i];
    for (int j = i + 1; j < 5; ++j) c[j] = c[j - 1] + 1;
    return 1;
}

void orc_basis(int8_t *table /* [256][8] */) {
    static const int mags[3] = {2, 6, 10};
    int rows = 0;
    int16_t tmp[256][8];
    /* product((2,6,10), repeat=8): first coordinate varies slowest */
    for (int idx = 0; idx < 6561; ++idx) {
        int digits[8], rest = idx, norm = 0;
        for (int j = 7; j >= 0; --j) { digits[j] = rest % 3; rest /= 3; }
        for (int j = 0; j < 8; ++j) norm += mags[digits[j]] * mags[digits[j]];
        if (norm > 160) continue;
        for (int j = 0; j < 8; ++j) tmp[rows][j] = (int16_t)mags[digits[j]];
        ++rows;
    }
    /* 29 outer rows: five 6s, three 2s, subset number i*56/29 */
    int subsets[56][5], c[5] = {0, 1, 2, 3, 4}, count = 0;
    do { memcpy(subsets[count++], c, sizeof c); } while (next_subset(c));
    for (int i = 0; i < 29; ++i) {
        for (int j = 0; j < 8; ++j) tmp[rows][j] = 2;
        for (int j = 0; j < 5; ++j) tmp[rows][subsets[i * count / 29][j]] = 6;
        ++rows;
    }
    for (int r = 0; r < 256; ++r) {
        int sum = 0;
        for (int j = 0; j < 8; ++j) sum += tmp[r][j];
        if ((sum / 4) % 2) tmp[r][7] = (int16_t)-tmp[r][7];
        for (int j = 0; j < 8; ++j) table[r * 8 + j] = (int8_t)tmp[r][j];
    }
}

void orc_decode(const int8_t *table, uint16_t code, int8_t *q /* [8] */) {
    unsigned u = code & 255u, p = 0;
    for (int b = 0; b < 8; ++b) p ^= (u >> b) & 1u;
    unsigned m = u ^ p;
    for (int j = 0; j < 8; ++j) {
        int t = table[(code >> 8) * 8 + j];
        q[j] = (int8_t)(((m >> SIGN_BITS[j]) & 1u ? -t : t) + (p ? -1 : 1));
    }
}

void orc_decode_all(const int8_t *table, const uint16_t *codes, int64_t n, int8_t *out) {
    for (int64_t i = 0; i < n; ++i) orc_decode(table, codes[i], out + 8 * i);
}

/* packed u32 [n][k/8] -> int8 [n][k], w = a*decode(lo) + b*decode(hi) */
void orc_q4_integers(const int8_t *table, const uint32_t *packed, int64_t n, int64_t k,
                     int a, int b, int8_t *w) {
    for (int64_t i = 0; i < n * (k / 8); ++i) {
        int8_t q0[8], q1[8];
        orc_decode(table, (uint16_t)(packed[i] & 0xffffu), q0);
        orc_decode(table, (uint16_t)(packed[i] >> 16), q1);
        for (int j = 0; j < 8; ++j) w[8 * i + j] = (int8_t)(a * q0[j] + b * q1[j]);
    }
}

/* acc[m][n] = sum_k a[m][k]*w[n][k], pure integer */
void orc_int_dot(const int8_t *a, const int8_t *w, int64_t m, int64_t n, int64_t k, int32_t *acc) {
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            int32_t s = 0;
            for (int64_t x = 0; x < k; ++x) s += (int32_t)a[i * k + x] * (int32_t)w[j * k + x];
            acc[i * n + j] = s;
        }
}

/* One fused Q4A8 GEMV/GEMM row block straight from codes (no materialised weights):
 * acc[m][n] over packed u32 [n][k/8]. Used as the timed scalar CPU baseline. */
void orc_q4_dot(const int8_t *table, const uint32_t *packed, const int8_t *a, int64_t m, int64_t n,
                int64_t k, int32_t *acc) {
    for (int64_t j = 0; j < n; ++j) {
        for (int64_t i = 0; i < m; ++i) acc[i * n + j] = 0;
        for (int64_t g = 0; g < k / 8; ++g) {
            int8_t q0[8], q1[8];
            uint32_t c = packed[j * (k / 8) + g];
            orc_decode(table, (uint16_t)(c & 0xffffu), q0);
            orc_decode(table, (uint16_t)(c >> 16), q1);
            for (int64_t i = 0; i < m; ++i) {
                int32_t s = 0;
                for (int x = 0; x < 8; ++x) s += (4 * q0[x] + q1[x]) * (int32_t)a[i * k + 8 * g + x];
                acc[i * n + j] += s;
            }
        }
    }
}

/* out fp32 = (float(acc) * ws) * as ; the caller casts to fp16 */
void orc_rescale(const int32_t *acc, const float *ws, const float *as, int64_t m, int64_t n, float *out) {
    for (int64_t i = 0; i < m; ++i)
        for (int64_t j = 0; j < n; ++j) {
            volatile float t = (float)acc[i * n + j] * ws[j];
            out[i * n + j] = t * as[i];
        }
}

/* x: fp16 values already widened to fp32; scale_out: the fp32 value BEFORE the fp16 cast
 * (the caller rounds it to fp16 and calls orc_a8_codes with the rounded value). */
void orc_a8_scale(const float *x, int64_t rows, int64_t k, float *scale_out) {
    for (int64_t r = 0; r < rows; ++r) {
        float amax = 0.f;
        for (int64_t j = 0; j < k; ++j) { float v = fabsf(x[r * k + j]); if (v > amax) amax = v; }
        float s = amax / 127.0f;
        const float floor_ = 5.9604644775390625e-08f; /* 2^-24 */
        if (s < floor_) s = floor_;
        scale_out[r] = amax > 0.f ? s : 1.0f;
    }
}

void orc_a8_codes(const float *x, const float *scale, int64_t rows, int64_t k, int8_t *q) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t j = 0; j < k; ++j) {
            float v = nearbyintf(x[r * k + j] / scale[r]); /* default mode: ties to even */
            if (v > 127.f) v = 127.f;
            if (v < -127.f) v = -127.f;
            q[r * k + j] = (int8_t)v;
        }
}
