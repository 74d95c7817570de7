// Shared device/host helpers for the gfx950 MX kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdio>
#include <string>

#include "catccos_mx.h"

namespace cmx {

// ---- error plumbing --------------------------------------------------------------------------
void set_error(const std::string& msg);

#define CMX_REQUIRE(cond, msg)                                             \
    do {                                                                   \
        if (!(cond)) {                                                     \
            ::cmx::set_error(std::string(__func__) + ": " + (msg));        \
            return CMX_EINVAL;                                             \
        }                                                                  \
    } while (0)

#define CMX_HIP(call)                                                                                   \
    do {                                                                                                \
        hipError_t e_ = (call);                                                                         \
        if (e_ != hipSuccess) {                                                                         \
            ::cmx::set_error(std::string(__func__) + ": " #call " -> " + hipGetErrorString(e_));        \
            return CMX_ERUNTIME;                                                                        \
        }                                                                                               \
    } while (0)

#define CMX_LAUNCH_CHECK()                                                                       \
    do {                                                                                         \
        hipError_t e_ = hipGetLastError();                                                       \
        if (e_ != hipSuccess) {                                                                  \
            ::cmx::set_error(std::string(__func__) + ": launch -> " + hipGetErrorString(e_));    \
            return CMX_ERUNTIME;                                                                 \
        }                                                                                        \
    } while (0)

// Each translation unit with kernels is a code object of its own, loaded on a device when one of its kernels is first
// looked up there.  cmx_init calls these so that no later launch -- possibly one inside a stream capture -- is the
// first to do so.  Each asks the runtime for the attributes of one kernel of its unit on the current device.
int preload_routing_kernels();
int preload_layout_kernels();
int preload_quant_kernels();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }
inline uint32_t round_up(uint32_t a, uint32_t b) { return ceil_div(a, b) * b; }
inline size_t round_up_sz(size_t a, size_t b) { return (a + b - 1) / b * b; }
// scale bytes per row: ceil(cols/32) rounded up to an even count
inline uint32_t scale_cols(uint32_t cols) { return round_up(ceil_div(cols, 32), 2); }

// ---- element format traits -------------------------------------------------------------------
constexpr int kEmaxE4M3 = 8;
constexpr int kEmaxE5M2 = 15;
constexpr int kEmaxE2M1 = 2;
constexpr int kEmaxE1M2 = 0;

#if defined(__HIPCC__)

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// fp32 -> bf16 bits, round-to-nearest-even (finite inputs; NaN -> quiet NaN)
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? ((u >> 16) | 0x40u) : r;
}

// Shared exponent of a block from the bf16 bit pattern of its amax (sign cleared):
// e = 0 if amax < 1e-12 else clamp(floor(log2 amax) - emax, -128, 127).
// 0x2B8D is the smallest bf16 that is >= 1e-12.
__device__ __forceinline__ int block_exp_from_bf16_amax(uint32_t amax_bits, int emax) {
    int e = (int)(amax_bits >> 7) - 127 - emax;
    e = e > 127 ? 127 : e;
    return amax_bits < 0x2B8Du ? 0 : e;
}

// E4M3 codes of |y| <= 448 by the hardware RNE cast (OCP e4m3fn on gfx950); two values per call.
__device__ __forceinline__ uint32_t cvt_pk_e4m3(float a, float b, uint32_t old, bool hi) {
    return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, false);
}
__device__ __forceinline__ uint32_t cvt_pk_e5m2(float a, float b, uint32_t old, bool hi) {
    return hi ? (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, true)
              : (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(a, b, (int)old, false);
}

__device__ __forceinline__ float clamp_abs(float y, float lim) { return fminf(fmaxf(y, -lim), lim); }

// Value of a positive E4M3 / E5M2 magnitude code (0..0x7E / 0..0x7B), exact.
__device__ __forceinline__ float e4m3_mag_value(uint32_t c) {
    uint32_t e = c >> 3, m = c & 7u;
    return e == 0 ? (float)m * 0.001953125f : __uint_as_float(((e + 120u) << 23) | (m << 20));
}
__device__ __forceinline__ float e5m2_mag_value(uint32_t c) {
    uint32_t e = c >> 2, m = c & 3u;
    return e == 0 ? (float)m * 1.52587890625e-05f : __uint_as_float(((e + 112u) << 23) | (m << 21));
}

// Nearest-table-value encode with ties to the smaller magnitude and -0 -> +0:
// start from the RNE code r of |y|, look at its two neighbours and apply
// pick_lower = (|y| - lower) <= (upper - |y|) exactly as a sorted-table search does.
template <bool E5M2>
__device__ __forceinline__ uint32_t fp8_lut_fixup(float y, uint32_t rne_code) {
    const uint32_t maxc = E5M2 ? 0x7Bu : 0x7Eu;
    float mag = fabsf(y);
    uint32_t r = rne_code & 0x7Fu;
    float vr = E5M2 ? e5m2_mag_value(r) : e4m3_mag_value(r);
    uint32_t lo, hi;
    if (vr >= mag) {
        hi = r;
        lo = r > 0 ? r - 1 : 0;
    } else {
        lo = r;
        hi = r < maxc ? r + 1 : maxc;
    }
    float vlo = E5M2 ? e5m2_mag_value(lo) : e4m3_mag_value(lo);
    float vhi = E5M2 ? e5m2_mag_value(hi) : e4m3_mag_value(hi);
    uint32_t c = ((mag - vlo) <= (vhi - mag)) ? lo : hi;
    return (c != 0 && y < 0.0f) ? (c | 0x80u) : c;
}

// E2M1 code of |y| <= 6.  LUT: ties to the smaller magnitude, -0 -> 0.  RNE: ties to the even
// mantissa bit, sign kept.
__device__ __forceinline__ uint32_t e2m1_encode(float y, bool lut) {
    float a = fabsf(y);
    uint32_t c;
    if (lut) {
        c = (a > 0.25f) + (a > 0.75f) + (a > 1.25f) + (a > 1.75f) + (a > 2.5f) + (a > 3.5f) + (a > 5.0f);
        return (c != 0 && y < 0.0f) ? (c | 8u) : c;
    }
    c = (a > 0.25f) + (a >= 0.75f) + (a > 1.25f) + (a >= 1.75f) + (a > 2.5f) + (a >= 3.5f) + (a > 5.0f);
    return c | ((__float_as_uint(y) >> 28) & 8u);
}

// E1M2 code of |y| <= 1.75: the grid is k / 4, k = 0..7 (one exponent bit, two mantissa bits, bias 1), same
// tie rules as E2M1.
__device__ __forceinline__ uint32_t e1m2_encode(float y, bool lut) {
    float a = fabsf(y);
    uint32_t c;
    if (lut) {
        c = (a > 0.125f) + (a > 0.375f) + (a > 0.625f) + (a > 0.875f) + (a > 1.125f) + (a > 1.375f) + (a > 1.625f);
        return (c != 0 && y < 0.0f) ? (c | 8u) : c;
    }
    c = (a > 0.125f) + (a >= 0.375f) + (a > 0.625f) + (a >= 0.875f) + (a > 1.125f) + (a >= 1.375f) + (a > 1.625f);
    return c | ((__float_as_uint(y) >> 28) & 8u);
}

template <int FMT>
__device__ __forceinline__ uint32_t fp4_encode(float y, bool lut) {
    return FMT == CMX_FMT_E1M2 ? e1m2_encode(y, lut) : e2m1_encode(y, lut);
}

// ---- packed 16-bit helpers (bf16 bit patterns) and the scaled hardware casts of gfx950 ----------------
typedef unsigned short v2u16 __attribute__((ext_vector_type(2)));
typedef short v2i16 __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf16 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2u16, a), __builtin_bit_cast(v2u16, b)));
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(v2u16, a), __builtin_bit_cast(v2u16, b)));
}

template <int FMT>
__device__ __forceinline__ uint32_t cvt_scaled_pk4(uint32_t d0, uint32_t d1, float scale) {
    v2i16 o = {0, 0};
    if constexpr (FMT == CMX_FMT_E4M3) {
        o = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, __builtin_bit_cast(v2bf16, d0), scale, false);
        o = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(o, __builtin_bit_cast(v2bf16, d1), scale, true);
    } else {
        o = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, __builtin_bit_cast(v2bf16, d0), scale, false);
        o = __builtin_amdgcn_cvt_scalef32_pk_bf8_bf16(o, __builtin_bit_cast(v2bf16, d1), scale, true);
    }
    return __builtin_bit_cast(uint32_t, o);
}

// Non-finite elements, which only a block whose maximum is Inf or NaN can hold (a rare branch behind the casts):
// Inf becomes the largest magnitude code with its sign, NaN the NaN code with its sign under the nearest-even cast
// and +0 under the table search -- what the reference's Python golden produces.  d = the block's eight bf16
// bit patterns of this lane, w0 / w1 = their eight codes.
template <int FMT, bool LUT>
__device__ __forceinline__ void patch_nonfinite_fp8(const uint32_t (&d)[4], uint32_t& w0, uint32_t& w1) {
    constexpr uint32_t maxc = FMT == CMX_FMT_E5M2 ? 0x7Bu : 0x7Eu;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t pat = (j & 1) ? d[j >> 1] >> 16 : d[j >> 1] & 0xFFFFu;
        const uint32_t mag = pat & 0x7FFFu;
        if (mag >= 0x7F80u) {
            const uint32_t sign = (pat >> 8) & 0x80u;
            const uint32_t code = mag == 0x7F80u ? (maxc | sign) : (LUT ? 0u : (0x7Fu | sign));
            const uint32_t sh = 8 * (j & 3);
            uint32_t& w = j < 4 ? w0 : w1;
            w = (w & ~(0xFFu << sh)) | (code << sh);
        }
    }
}

typedef float v2f32 __attribute__((ext_vector_type(2)));
// two floats -> packed bf16 (a in the low half), round-to-nearest-even in hardware
__device__ __forceinline__ uint32_t cvt_pk_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((v2f32){a, b}, v2bf16));
}

#endif  // __HIPCC__

}  // namespace cmx
