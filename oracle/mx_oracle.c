/*
 * CPU oracle in plain C (TEST INFRASTRUCTURE - never linked into or called by the product).
 *
 * A second, independent restatement of the integer/byte parts of the reference's golden path,
 * used to cross-check the numpy oracle and as a fast checker at full sizes.  Reference files
 * (relative to the reference checkout):
 *   E8M0 exponent            examples/utils/gen_mx_quant_allgather_data.py:168-189
 *   FP8 block quantizer      examples/utils/gen_mx_quant_allgather_data.py:255-313 (native = RNE, lut = ties down)
 *   FP4 block quantizer      examples/utils/gen_mx_quant_allgather_data.py:385-449
 *   routing sort             examples/utils/gen_data_moe.py:48-57, aux_ops/moe_init_routing_v2/moe_v2_src_to_dst_op_simt.h:79-87
 *   weighted combine         examples/aux_ops/moe_token_unpermute/moe_token_unpermute.h:233-366
 *   dequant + fp32 matmul    examples/utils/gen_data_moe.py:646-651
 * Formats: 0 = E4M3, 1 = E5M2, 2 = E2M1 (codes returned one per byte, unpacked).  Modes: 0 = RNE, 1 = LUT.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if (f != f) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

/* value of the positive magnitude code c of an 8-bit float with `man` mantissa bits and bias `bias` */
static double fp8_value(int c, int man, int bias) {
    int e = c >> man, m = c & ((1 << man) - 1);
    if (e == 0) return ldexp((double)m, 1 - bias - man);
    return ldexp(1.0 + (double)m / (1 << man), e - bias);
}

static int signbit_of(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return (int)(u >> 31);
}

static const double kFp4[8] = {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0};

/* nearest code of |y| among codes 0..maxc; ties: rne -> even code, lut -> smaller magnitude */
static int nearest_code(double mag, int maxc, int fmt, int lut) {
    int best = 0;
    double bestd = INFINITY;
    for (int c = 0; c <= maxc; ++c) {
        double v = fmt == 2 ? kFp4[c] : (fmt == 0 ? fp8_value(c, 3, 7) : fp8_value(c, 2, 15));
        double d = fabs(v - mag);
        if (d < bestd || (!lut && d == bestd && (c & 1) == 0)) {
            best = c;
            bestd = d;
        }
    }
    return best;
}

static int block_exp(float amax, int emax) {
    if (amax < 1e-12f) return 0;
    uint32_t u;
    memcpy(&u, &amax, 4);
    int e = (int)((u >> 23) & 0xFF) - 127 - emax;
    if (e < -128) e = -128;
    if (e > 127) e = 127;
    return e;
}

int mxo_scale_cols(int cols) {
    int nb = (cols + 31) / 32;
    return (nb + 1) / 2 * 2;
}

/* x bf16 [rows, cols] -> codes u8 [rows, cols] (one code per byte), scales u8 [rows, mxo_scale_cols(cols)] */
int mxo_quant_bf16(const uint16_t* x, int rows, int cols, int fmt, int mode, uint8_t* codes, uint8_t* scales) {
    static const int emaxs[3] = {8, 15, 2};
    static const double maxv[3] = {448.0, 57344.0, 6.0};
    static const int maxc[3] = {0x7E, 0x7B, 7};
    if (fmt < 0 || fmt > 2 || (mode != 0 && mode != 1)) return -1;
    const int nb = (cols + 31) / 32, sc = mxo_scale_cols(cols);
    const int signbit = fmt == 2 ? 8 : 0x80;
    for (int r = 0; r < rows; ++r) {
        for (int b = 0; b < sc; ++b) scales[(size_t)r * sc + b] = 127;
        for (int b = 0; b < nb; ++b) {
            const int lo = b * 32, hi = lo + 32 < cols ? lo + 32 : cols;
            float amax = 0.0f;
            int has_nan = 0;
            for (int c = lo; c < hi; ++c) {
                float a = fabsf(bf16_to_f32(x[(size_t)r * cols + c]));
                if (a != a) has_nan = 1;
                if (a > amax) amax = a;
            }
            /* A maximum of Inf or NaN, as the golden treats it (torch's amax returns NaN if the block holds one):
             * the 8-bit path reads the exponent field, 255, of either (:181-189); the 4-bit path takes
             * floor(log2(.)) in floating point (:429-432): Inf -> the largest exponent, NaN -> a NaN scale
             * (byte 255) that makes every quotient NaN and every code 0. */
            int e = block_exp(amax, emaxs[fmt]);
            if (fmt != 2 && (has_nan || isinf(amax))) e = 128 - emaxs[fmt];
            if (fmt == 2 && isinf(amax)) e = 127;
            const int nan_scale = fmt == 2 && has_nan;
            scales[(size_t)r * sc + b] = nan_scale ? 255 : (uint8_t)(e + 127);
            for (int c = lo; c < hi; ++c) {
                const float xv = bf16_to_f32(x[(size_t)r * cols + c]);
                if (nan_scale) {
                    codes[(size_t)r * cols + c] = 0;
                    continue;
                }
                if (xv != xv) {         /* NaN element: NaN code with its sign under the cast, +0 under the table search */
                    codes[(size_t)r * cols + c] = (fmt != 2 && mode == 0) ? (uint8_t)(0x7F | (signbit_of(xv) ? 0x80 : 0)) : 0;
                    continue;
                }
                double y = ldexp((double)xv, -e);
                if (y > maxv[fmt]) y = maxv[fmt];
                if (y < -maxv[fmt]) y = -maxv[fmt];
                const int code = nearest_code(fabs(y), maxc[fmt], fmt, mode);
                const int neg = mode == 1 ? (y < 0 && code != 0) : signbit_of(xv);
                codes[(size_t)r * cols + c] = (uint8_t)(code | (neg ? signbit : 0));
            }
        }
    }
    return 0;
}

void mxo_dequant(const uint8_t* codes, const uint8_t* scales, int rows, int cols, int fmt, float* out) {
    const int sc = mxo_scale_cols(cols);
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            const int code = codes[(size_t)r * cols + c];
            double v;
            if (fmt == 2) {
                v = kFp4[code & 7];
                if (code & 8) v = -v;
            } else {
                int m = code & 0x7F;
                if (fmt == 0) v = m == 0x7F ? 448.0 : fp8_value(m, 3, 7);
                else v = m >= 0x7C ? 57344.0 : fp8_value(m, 2, 15);
                if (code & 0x80) v = -v;
            }
            out[(size_t)r * cols + c] = (float)ldexp(v, (int)scales[(size_t)r * sc + c / 32] - 127);
        }
}

/* c[m, n] = sum_k a[m, k] * b[n, k], fp32 operands, double accumulation (a tolerance-level golden) */
void mxo_gemm_nt(const float* a, const float* b, int m, int n, int k, float* c) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0.0;
            for (int t = 0; t < k; ++t) s += (double)a[(size_t)i * k + t] * (double)b[(size_t)j * k + t];
            c[(size_t)i * n + j] = (float)s;
        }
}

/* stable counting sort of the flattened expert ids; ids outside [0, experts) are rejected */
int mxo_routing(const int32_t* idx, int routes, int experts, int32_t* sorted2src, int32_t* src2sorted, int32_t* counts) {
    int64_t* start = (int64_t*)calloc((size_t)experts + 1, sizeof(int64_t));
    if (!start) return -2;
    for (int e = 0; e < experts; ++e) counts[e] = 0;
    for (int i = 0; i < routes; ++i) {
        if (idx[i] < 0 || idx[i] >= experts) {
            free(start);
            return -1;
        }
        counts[idx[i]]++;
    }
    for (int e = 0; e < experts; ++e) start[e + 1] = start[e] + counts[e];
    for (int i = 0; i < routes; ++i) {
        const int64_t pos = start[idx[i]]++;
        sorted2src[pos] = i;
        src2sorted[i] = (int32_t)pos;
    }
    free(start);
    return 0;
}

/* out[t] = bf16( sum_k probs[t,k] * y[src2sorted[t*topk+k]] ): fp32 multiply, then fp32 add, in k order */
void mxo_combine(const uint16_t* y, int rows, int hidden, const int32_t* src2sorted, const float* probs, int tokens,
                 int topk, uint16_t* out) {
    for (int t = 0; t < tokens; ++t)
        for (int c = 0; c < hidden; ++c) {
            volatile float acc = 0.0f;
            for (int k = 0; k < topk; ++k) {
                const int32_t r = src2sorted[(size_t)t * topk + k];
                volatile float term = 0.0f;
                if (r >= 0 && r < rows) term = bf16_to_f32(y[(size_t)r * hidden + c]) * probs[(size_t)t * topk + k];
                if (k == 0) acc = term; else acc = acc + term;
            }
            out[(size_t)t * hidden + c] = f32_to_bf16(acc);
        }
}
