// MX block-32 quantizer for gfx950: bf16 rows -> E4M3 / E5M2 / E2M1 / E1M2 codes + E8M0 scales.
//
// Work split: four adjacent lanes own one 32-element block (8 bf16 = one 16-byte load each), so a
// wavefront reads 1 KiB of contiguous input per step and every lane keeps UNROLL loads in flight.
// The block amax is an integer max over sign-cleared bf16 bit patterns, reduced across the four
// lanes with two DPP quad permutes; the shared exponent comes straight from the amax's exponent
// field.  Elements are scaled by an exact power of two (ldexp), clamped to the format's range
// and cast by the hardware RNE converters; the table-rounding mode patches exact ties afterwards.
#include "mx_common.h"

namespace cmx {

namespace {

constexpr int kUnroll = 4;
constexpr int kThreads = 256;
constexpr int kBlocksPerIter = kThreads / 4;   // MX blocks handled per unroll step by one workgroup

__device__ __forceinline__ uint32_t quad_max(uint32_t v) {
    // quad_perm [1,0,3,2] then [2,3,0,1]
    uint32_t t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);
    v = v > t ? v : t;
    t = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);
    return v > t ? v : t;
}

template <int FMT, bool LUT>
__global__ __launch_bounds__(kThreads) void mx_quant_kernel(const uint16_t* __restrict__ x, uint32_t ld_x,
                                                            uint8_t* __restrict__ codes, uint32_t ld_codes,
                                                            uint8_t* __restrict__ scales, uint32_t ld_scales,
                                                            uint32_t rows, uint32_t cols, uint32_t nb,
                                                            uint32_t total_blocks, int vec_in, int vec_out) {
    constexpr bool kFp4 = FMT == CMX_FMT_E2M1 || FMT == CMX_FMT_E1M2;
    constexpr int emax = FMT == CMX_FMT_E4M3 ? kEmaxE4M3 : (FMT == CMX_FMT_E5M2 ? kEmaxE5M2 : (FMT == CMX_FMT_E2M1 ? kEmaxE2M1 : kEmaxE1M2));
    constexpr float lim = FMT == CMX_FMT_E4M3 ? 448.0f : (FMT == CMX_FMT_E5M2 ? 57344.0f : (FMT == CMX_FMT_E2M1 ? 6.0f : 1.75f));
    const uint32_t q = threadIdx.x & 3u;
    const uint32_t b0 = blockIdx.x * (kBlocksPerIter * kUnroll) + (threadIdx.x >> 2);

    uint4 raw[kUnroll];
    uint32_t row_[kUnroll], kb_[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        uint32_t b = b0 + u * kBlocksPerIter;
        bool live = b < total_blocks;
        uint32_t row = live ? b / nb : 0;
        uint32_t kb = live ? b - row * nb : 0;
        row_[u] = row;
        kb_[u] = kb;
        uint32_t col = kb * 32 + q * 8;
        raw[u] = make_uint4(0, 0, 0, 0);
        if (live) {
            const uint16_t* p = x + (size_t)row * ld_x + col;
            if (vec_in) {
                if (col < cols) raw[u] = *reinterpret_cast<const uint4*>(p);
            } else {
                uint32_t w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = (col + i < cols) ? p[i] : 0u;
                raw[u] = make_uint4(w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16), w[6] | (w[7] << 16));
            }
        }
    }

#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        uint32_t b = b0 + u * kBlocksPerIter;
        bool live = b < total_blocks;
        uint32_t d[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
        uint32_t amax = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t a = d[i] & 0x7FFF7FFFu;
            uint32_t lo = a & 0xFFFFu, hi = a >> 16;
            amax = amax > lo ? amax : lo;
            amax = amax > hi ? amax : hi;
        }
        amax = quad_max(amax);
        int e = block_exp_from_bf16_amax(amax, emax);
        // a block whose maximum is Inf or NaN: the 8-bit formats take the exponent field as it is (255), the 4-bit
        // formats the largest exponent for Inf and a NaN scale (byte 255, every code 0) for NaN
        const bool nonfinite = amax >= 0x7F80u;
        if (kFp4 && nonfinite) e = 127;

        float y[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            y[2 * i] = clamp_abs(ldexpf(__uint_as_float(d[i] << 16), -e), lim);
            y[2 * i + 1] = clamp_abs(ldexpf(__uint_as_float(d[i] & 0xFFFF0000u), -e), lim);
        }
        if (!live) continue;
        const uint32_t row = row_[u], kb = kb_[u];
        const uint32_t col = kb * 32 + q * 8;

        if constexpr (kFp4) {
            uint32_t pk = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) pk |= fp4_encode<FMT>(y[i], LUT) << (4 * i);
            if (amax > 0x7F80u) pk = 0;
            uint8_t* o = codes + (size_t)row * ld_codes + (col >> 1);
            if (vec_out) {
                if (col < cols) *reinterpret_cast<uint32_t*>(o) = pk;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (col + 2 * i < cols) o[i] = (uint8_t)(pk >> (8 * i));
            }
        } else {
            uint32_t w0 = 0, w1 = 0;
            if constexpr (FMT == CMX_FMT_E4M3) {
                w0 = cvt_pk_e4m3(y[0], y[1], w0, false);
                w0 = cvt_pk_e4m3(y[2], y[3], w0, true);
                w1 = cvt_pk_e4m3(y[4], y[5], w1, false);
                w1 = cvt_pk_e4m3(y[6], y[7], w1, true);
            } else {
                w0 = cvt_pk_e5m2(y[0], y[1], w0, false);
                w0 = cvt_pk_e5m2(y[2], y[3], w0, true);
                w1 = cvt_pk_e5m2(y[4], y[5], w1, false);
                w1 = cvt_pk_e5m2(y[6], y[7], w1, true);
            }
            if constexpr (LUT) {
                uint32_t f0 = 0, f1 = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    f0 |= fp8_lut_fixup<FMT == CMX_FMT_E5M2>(y[i], (w0 >> (8 * i)) & 0xFFu) << (8 * i);
                    f1 |= fp8_lut_fixup<FMT == CMX_FMT_E5M2>(y[4 + i], (w1 >> (8 * i)) & 0xFFu) << (8 * i);
                }
                w0 = f0;
                w1 = f1;
            }
            if (nonfinite) patch_nonfinite_fp8<FMT, LUT>(d, w0, w1);
            uint8_t* o = codes + (size_t)row * ld_codes + col;
            if (vec_out) {
                if (col < cols) *reinterpret_cast<uint2*>(o) = make_uint2(w0, w1);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (col + i < cols) o[i] = (uint8_t)(w0 >> (8 * i));
                    if (col + 4 + i < cols) o[4 + i] = (uint8_t)(w1 >> (8 * i));
                }
            }
        }
        if (q == 0) {
            uint8_t* s = scales + (size_t)row * ld_scales;
            s[kb] = (kFp4 && amax > 0x7F80u) ? (uint8_t)255 : (uint8_t)(e + 127);
            if (kb == nb - 1 && (nb & 1u) && ld_scales > nb) s[nb] = 127;   // pad the scale row to an even count with 1.0
        }
    }
}

// ---- fast path: RNE 8-bit formats, cols % 32 == 0, 16-byte aligned rows ------------------------
// Same lane split (four lanes per block, one 16-byte load each) but laid out so that no lane ever
// divides: a workgroup owns 64 consecutive blocks of four consecutive rows, one row per unroll step.
// The arithmetic stays on packed 16-bit integers until the final cast: amax and the clamp to
// +-max_normal * 2^e work on sign-cleared bf16 bit patterns (unsigned order == magnitude order), and
// v_cvt_scalef32_pk_{fp8,bf8}_bf16 divides by 2^e and rounds to nearest even in one instruction.
// Each lane of a quad then stores the scale byte of one of the four rows.
constexpr int kFastRows = 4;

template <int FMT>
__global__ __launch_bounds__(kThreads) void mx_quant_rne8_kernel(const uint8_t* __restrict__ x, uint32_t ld_x_bytes,
                                                                 uint8_t* __restrict__ codes, uint32_t ld_codes,
                                                                 uint8_t* __restrict__ scales, uint32_t ld_scales,
                                                                 uint32_t rows, uint32_t nb) {
    constexpr int emax = FMT == CMX_FMT_E4M3 ? kEmaxE4M3 : kEmaxE5M2;
    constexpr uint32_t lim_mant = FMT == CMX_FMT_E4M3 ? 0x60u : 0x60u;   // 448 = 1.75 * 2^8, 57344 = 1.75 * 2^15
    const uint32_t q = threadIdx.x & 3u;
    const uint32_t kb = blockIdx.x * kBlocksPerIter + (threadIdx.x >> 2);
    const uint32_t row0 = blockIdx.y * kFastRows;
    if (kb >= nb) return;                                  // whole quads leave together
    const uint32_t in_off = kb * 64u + q * 16u;            // bytes inside the row
    const uint32_t out_off = kb * 32u + q * 8u;

    uint4 raw[kFastRows];
#pragma unroll
    for (int u = 0; u < kFastRows; ++u) {
        const uint32_t row = row0 + u;
        raw[u] = make_uint4(0, 0, 0, 0);
        if (row < rows) raw[u] = *reinterpret_cast<const uint4*>(x + (size_t)row * ld_x_bytes + in_off);
    }
    int my_e = 0;
#pragma unroll
    for (int u = 0; u < kFastRows; ++u) {
        const uint32_t row = row0 + u;
        const uint32_t d[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
        uint32_t a[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = d[i] & 0x7FFF7FFFu;
        uint32_t m = pk_max_u16(pk_max_u16(a[0], a[1]), pk_max_u16(a[2], a[3]));
        m = pk_max_u16(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));
        m = pk_max_u16(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xF, 0xF, true));
        const uint32_t amax = max(m & 0xFFFFu, m >> 16);
        const int e = block_exp_from_bf16_amax(amax, emax);
        // clamp magnitudes to max_normal * 2^e (bit pattern: exponent e + emax + 127, mantissa 1.75)
        const uint32_t lim = (((uint32_t)(e + emax + 127) << 7) | lim_mant) * 0x10001u;
        const float scale = __uint_as_float((uint32_t)(e + 127) << 23);
        uint32_t c[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) c[i] = pk_min_u16(a[i], lim) | (d[i] & 0x80008000u);
        uint32_t w0 = cvt_scaled_pk4<FMT>(c[0], c[1], scale);
        uint32_t w1 = cvt_scaled_pk4<FMT>(c[2], c[3], scale);
        if (amax >= 0x7F80u) patch_nonfinite_fp8<FMT, false>(d, w0, w1);      // Inf / NaN in the block (rare)
        if (row < rows) *reinterpret_cast<uint2*>(codes + (size_t)row * ld_codes + out_off) = make_uint2(w0, w1);
        my_e = (int)q == u ? e : my_e;
    }
    const uint32_t srow = row0 + q;
    if (srow < rows) {
        uint8_t* sp = scales + (size_t)srow * ld_scales;
        sp[kb] = (uint8_t)(my_e + 127);
        if (kb == nb - 1 && (nb & 1u) && ld_scales > nb) sp[nb] = 127;       // pad the scale row to an even count with 1.0
    }
}

__global__ void mx_dequant_kernel(const uint8_t* __restrict__ codes, uint32_t ld_codes,
                                  const uint8_t* __restrict__ scales, uint32_t ld_scales, float* __restrict__ out,
                                  uint32_t ld_out, uint32_t rows, uint32_t cols, int fmt) {
    uint32_t col = blockIdx.y * blockDim.x + threadIdx.x;
    uint32_t row = blockIdx.x;
    if (col >= cols || row >= rows) return;
    int e = (int)scales[(size_t)row * ld_scales + (col >> 5)] - 127;
    float v;
    if (fmt == CMX_FMT_E2M1 || fmt == CMX_FMT_E1M2) {
        uint32_t byte = codes[(size_t)row * ld_codes + (col >> 1)];
        uint32_t c = (col & 1u) ? (byte >> 4) : (byte & 0xFu);
        const float tab[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
        v = fmt == CMX_FMT_E2M1 ? tab[c & 7u] : 0.25f * (float)(c & 7u);
        if (c & 8u) v = -v;
    } else {
        uint32_t c = codes[(size_t)row * ld_codes + col];
        uint32_t m = c & 0x7Fu;
        if (fmt == CMX_FMT_E4M3) {
            v = m == 0x7Fu ? 448.0f : e4m3_mag_value(m);
        } else {
            v = m >= 0x7Cu ? 57344.0f : e5m2_mag_value(m);
        }
        if (c & 0x80u) v = -v;
    }
    out[(size_t)row * ld_out + col] = ldexpf(v, e);
}

template <int FMT>
int launch_quant(bool lut, dim3 grid, hipStream_t s, const uint16_t* x, uint32_t ld_x, uint8_t* codes,
                 uint32_t ld_codes, uint8_t* scales, uint32_t ld_scales, uint32_t rows, uint32_t cols, uint32_t nb,
                 uint32_t total, int vec_in, int vec_out) {
    if (lut)
        hipLaunchKernelGGL((mx_quant_kernel<FMT, true>), grid, dim3(kThreads), 0, s, x, ld_x, codes, ld_codes, scales,
                           ld_scales, rows, cols, nb, total, vec_in, vec_out);
    else
        hipLaunchKernelGGL((mx_quant_kernel<FMT, false>), grid, dim3(kThreads), 0, s, x, ld_x, codes, ld_codes,
                           scales, ld_scales, rows, cols, nb, total, vec_in, vec_out);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

}  // namespace

}  // namespace cmx

int cmx::preload_quant_kernels() {
    hipFuncAttributes attr;
    CMX_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(cmx::mx_dequant_kernel)));
    return CMX_OK;
}

extern "C" int cmx_mx_quant(const void* x, uint32_t ld_x, uint8_t* codes, uint32_t ld_codes, uint8_t* scales,
                            uint32_t ld_scales, uint32_t rows, uint32_t cols, int fmt, int round_mode,
                            cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(x && codes && scales, "null pointer");
    CMX_REQUIRE(fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2 || fmt == CMX_FMT_E2M1 || fmt == CMX_FMT_E1M2, "unknown element format");
    CMX_REQUIRE(round_mode == CMX_ROUND_RNE || round_mode == CMX_ROUND_LUT, "unknown rounding mode");
    if (rows == 0 || cols == 0) return CMX_OK;
    const uint32_t nb = ceil_div(cols, 32);
    const bool fp4 = fmt == CMX_FMT_E2M1 || fmt == CMX_FMT_E1M2;
    const uint32_t code_cols = fp4 ? ceil_div(cols, 2) : cols;
    // a scale pitch of exactly ceil(cols / 32) columns selects the unpadded scale rows of the reference's
    // mx_quant_allgather files; any larger pitch must hold the even-padded row
    CMX_REQUIRE(ld_x >= cols && ld_codes >= code_cols && (ld_scales == nb || ld_scales >= scale_cols(cols)), "row pitch smaller than row");
    CMX_REQUIRE((uint64_t)rows * nb < (1ull << 32), "too many blocks for one launch");
    const uint32_t total = rows * nb;
    const int vec_in = (cols % 8 == 0) && (ld_x % 8 == 0) && aligned16(x);
    const int vec_out = (cols % 8 == 0) && (ld_codes % 8 == 0) && ((reinterpret_cast<uintptr_t>(codes) & 7u) == 0);
    dim3 grid(ceil_div(total, kBlocksPerIter * kUnroll));
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const bool lut = round_mode == CMX_ROUND_LUT;
    const bool fast = !lut && !fp4 && cols % 32 == 0 && vec_in && vec_out &&
                      (uint64_t)ld_x * 2 < (1ull << 32) && ceil_div(rows, kFastRows) <= 65535u;
    if (fast) {
        dim3 fgrid(ceil_div(nb, kBlocksPerIter), ceil_div(rows, kFastRows));
        const uint8_t* xb = static_cast<const uint8_t*>(x);
        if (fmt == CMX_FMT_E4M3)
            hipLaunchKernelGGL((mx_quant_rne8_kernel<CMX_FMT_E4M3>), fgrid, dim3(kThreads), 0, s, xb, ld_x * 2, codes, ld_codes,
                               scales, ld_scales, rows, nb);
        else
            hipLaunchKernelGGL((mx_quant_rne8_kernel<CMX_FMT_E5M2>), fgrid, dim3(kThreads), 0, s, xb, ld_x * 2, codes, ld_codes,
                               scales, ld_scales, rows, nb);
        CMX_LAUNCH_CHECK();
        return CMX_OK;
    }
    switch (fmt) {
        case CMX_FMT_E4M3:
            return launch_quant<CMX_FMT_E4M3>(lut, grid, s, xp, ld_x, codes, ld_codes, scales, ld_scales, rows, cols, nb,
                                              total, vec_in, vec_out);
        case CMX_FMT_E5M2:
            return launch_quant<CMX_FMT_E5M2>(lut, grid, s, xp, ld_x, codes, ld_codes, scales, ld_scales, rows, cols, nb,
                                              total, vec_in, vec_out);
        case CMX_FMT_E2M1:
            return launch_quant<CMX_FMT_E2M1>(lut, grid, s, xp, ld_x, codes, ld_codes, scales, ld_scales, rows, cols, nb,
                                              total, vec_in, vec_out);
        default:
            return launch_quant<CMX_FMT_E1M2>(lut, grid, s, xp, ld_x, codes, ld_codes, scales, ld_scales, rows, cols, nb,
                                              total, vec_in, vec_out);
    }
}

extern "C" int cmx_mx_dequant(const uint8_t* codes, uint32_t ld_codes, const uint8_t* scales, uint32_t ld_scales,
                              float* out, uint32_t ld_out, uint32_t rows, uint32_t cols, int fmt,
                              cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(codes && scales && out, "null pointer");
    CMX_REQUIRE(fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2 || fmt == CMX_FMT_E2M1 || fmt == CMX_FMT_E1M2, "unknown element format");
    if (rows == 0 || cols == 0) return CMX_OK;
    CMX_REQUIRE(ceil_div(cols, 256) <= 65535u, "too many columns for the debug dequantizer");
    dim3 grid(rows, ceil_div(cols, 256));
    hipLaunchKernelGGL(mx_dequant_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), codes, ld_codes,
                       scales, ld_scales, out, ld_out, rows, cols, fmt);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}
