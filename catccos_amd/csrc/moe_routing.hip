// MoE routing on one device: stable counting sort of (expert, route) pairs, fused MX quantise +
// scatter of the routed rows, and the weighted top-k combine.  All three are HBM-bound.
//
// Sort = histogram per 512-route chunk -> one-workgroup scan (expert-major, chunk-minor, which is
// exactly the order of a stable sort) -> scatter, where each chunk is owned by one wavefront that
// ranks equal keys in lane order with ballots, so the result is the unique stable permutation with
// no global atomics and no dependence on scheduling.
#include "mx_common.h"

namespace cmx {
namespace {

constexpr uint32_t kChunk = 512;   // routes per wavefront-owned chunk

__global__ __launch_bounds__(64) void route_hist_kernel(const int32_t* __restrict__ keys, uint32_t routes,
                                                         uint32_t experts, uint32_t* __restrict__ hist) {
    extern __shared__ uint32_t sh[];
    for (uint32_t e = threadIdx.x; e < experts; e += 64) sh[e] = 0;
    __syncthreads();
    const uint32_t base = blockIdx.x * kChunk;
    for (uint32_t i = threadIdx.x; i < kChunk; i += 64) {
        const uint32_t r = base + i;
        if (r < routes) {
            const int32_t k = keys[r];
            if (k >= 0 && (uint32_t)k < experts) atomicAdd(&sh[k], 1u);
        }
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < experts; e += 64) hist[(size_t)blockIdx.x * experts + e] = sh[e];
}

// hist[c][e] -> offset[c][e] = (rows of experts < e) + (rows of expert e in chunks < c); counts[e].
__global__ __launch_bounds__(1024) void route_scan_kernel(uint32_t* __restrict__ hist, uint32_t chunks, uint32_t experts,
                                                           int32_t* __restrict__ counts) {
    extern __shared__ uint32_t sh[];            // [experts] totals, then [1024] partials
    uint32_t* tot = sh;
    uint32_t* part = sh + experts;
    for (uint32_t e = threadIdx.x; e < experts; e += blockDim.x) {
        // the column walk is latency bound: fetch eight chunk counts at a time before touching the running sum
        uint32_t run = 0;
        uint32_t c = 0;
        for (; c + 8 <= chunks; c += 8) {
            uint32_t h[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = hist[(size_t)(c + i) * experts + e];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                hist[(size_t)(c + i) * experts + e] = run;
                run += h[i];
            }
        }
        for (; c < chunks; ++c) {
            const uint32_t h = hist[(size_t)c * experts + e];
            hist[(size_t)c * experts + e] = run;
            run += h;
        }
        tot[e] = run;
        counts[e] = (int32_t)run;
    }
    __syncthreads();
    // exclusive scan of tot[] over experts: contiguous segment per thread + scan of the partials
    const uint32_t seg = (experts + blockDim.x - 1) / blockDim.x;
    const uint32_t lo = threadIdx.x * seg;
    uint32_t s = 0;
    for (uint32_t e = lo; e < lo + seg && e < experts; ++e) s += tot[e];
    part[threadIdx.x] = s;
    __syncthreads();
    for (uint32_t d = 1; d < blockDim.x; d <<= 1) {
        uint32_t v = threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    uint32_t run = threadIdx.x ? part[threadIdx.x - 1] : 0;
    for (uint32_t e = lo; e < lo + seg && e < experts; ++e) {
        const uint32_t t = tot[e];
        tot[e] = run;
        run += t;
    }
    __syncthreads();
    for (uint32_t e = threadIdx.x; e < experts; e += blockDim.x) {
        const uint32_t b = tot[e];
        uint32_t c = 0;
        for (; c + 8 <= chunks; c += 8) {
            uint32_t h[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = hist[(size_t)(c + i) * experts + e];
#pragma unroll
            for (int i = 0; i < 8; ++i) hist[(size_t)(c + i) * experts + e] = h[i] + b;
        }
        for (; c < chunks; ++c) hist[(size_t)c * experts + e] += b;
    }
}

__global__ __launch_bounds__(64) void route_scatter_kernel(const int32_t* __restrict__ keys, uint32_t routes,
                                                            uint32_t experts, uint32_t key_bits,
                                                            const uint32_t* __restrict__ offset,
                                                            int32_t* __restrict__ sorted2src,
                                                            int32_t* __restrict__ src2sorted) {
    extern __shared__ uint32_t off[];
    const uint32_t lane = threadIdx.x;
    for (uint32_t e = lane; e < experts; e += 64) off[e] = offset[(size_t)blockIdx.x * experts + e];
    __syncthreads();
    const uint32_t base = blockIdx.x * kChunk;
    for (uint32_t i = 0; i < kChunk; i += 64) {
        const uint32_t r = base + i + lane;
        int32_t k = -1;
        if (r < routes) {
            k = keys[r];
            if (k < 0 || (uint32_t)k >= experts) k = -1;
        }
        const bool live = k >= 0;
        unsigned long long same = __ballot(live);
        for (uint32_t b = 0; b < key_bits; ++b) {
            const unsigned long long m = __ballot(live && ((k >> b) & 1));
            same &= ((k >> b) & 1) ? m : ~m;
        }
        if (live) {
            const uint32_t rank = __popcll(same & ((1ull << lane) - 1ull));
            const uint32_t pos = off[k] + rank;
            sorted2src[pos] = (int32_t)r;
            src2sorted[r] = (int32_t)pos;
        } else if (r < routes) {
            src2sorted[r] = -1;
        }
        __syncthreads();
        if (live && lane == 63u - (uint32_t)__clzll(same)) off[k] += (uint32_t)__popcll(same);
        __syncthreads();
    }
}

// ---- fused quantise + scatter -------------------------------------------------------------------

// Two lanes per MX block: each takes 16 elements with two 16-byte loads issued together, so a destination row is
// written 16 bytes per lane, 1 KiB per wavefront and store instruction.  A workgroup owns 128 consecutive blocks.
// The destination rows of the token are read before the arithmetic, eight at a time.  When scale rows hold whole
// dwords (VEC_SCALES: k a multiple of 128, dword-aligned scale rows) the scale bytes of four neighbouring blocks
// travel in one dword store instead of four byte stores.  k % 32 == 0, rows 16-byte aligned.
template <bool VEC_SCALES>
__global__ __launch_bounds__(256) void quant_scatter_kernel(const uint16_t* __restrict__ x, uint32_t ld_x,
                                                             const int32_t* __restrict__ src2sorted,
                                                             uint8_t* __restrict__ out_codes, uint32_t ld_out,
                                                             uint8_t* __restrict__ out_scales, uint32_t ld_outs,
                                                             uint32_t tokens, uint32_t k, uint32_t top_k, uint32_t nb,
                                                             uint32_t total_blocks) {
    const uint32_t h = threadIdx.x & 1u;
    const uint32_t b = blockIdx.x * 128 + (threadIdx.x >> 1);
    const bool live = b < total_blocks;
    const uint32_t row = live ? b / nb : 0;
    const uint32_t kb = live ? b - row * nb : 0;
    const uint32_t col = kb * 32 + h * 16;
    uint4 raw0 = make_uint4(0, 0, 0, 0), raw1 = raw0;
    if (live) {
        const uint16_t* src = x + (size_t)row * ld_x + col;
        raw0 = *reinterpret_cast<const uint4*>(src);
        raw1 = *reinterpret_cast<const uint4*>(src + 8);
    }
    int32_t dst[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[j] = (live && (uint32_t)j < top_k) ? src2sorted[(size_t)row * top_k + j] : -1;
    // amax, clamp and cast on packed bf16 bit patterns, as in the stand-alone quantizer's fast path
    const uint32_t d0[4] = {raw0.x, raw0.y, raw0.z, raw0.w}, d1[4] = {raw1.x, raw1.y, raw1.z, raw1.w};
    uint32_t a0[4], a1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a0[i] = d0[i] & 0x7FFF7FFFu;
        a1[i] = d1[i] & 0x7FFF7FFFu;
    }
    uint32_t m = pk_max_u16(pk_max_u16(pk_max_u16(a0[0], a0[1]), pk_max_u16(a0[2], a0[3])),
                            pk_max_u16(pk_max_u16(a1[0], a1[1]), pk_max_u16(a1[2], a1[3])));
    m = pk_max_u16(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));      // the block's other lane
    const uint32_t amax = max(m & 0xFFFFu, m >> 16);
    const int e = block_exp_from_bf16_amax(amax, kEmaxE4M3);
    const uint32_t lim = (((uint32_t)(e + kEmaxE4M3 + 127) << 7) | 0x60u) * 0x10001u;
    const float scale = __uint_as_float((uint32_t)(e + 127) << 23);
    uint32_t c0[4], c1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        c0[i] = pk_min_u16(a0[i], lim) | (d0[i] & 0x80008000u);
        c1[i] = pk_min_u16(a1[i], lim) | (d1[i] & 0x80008000u);
    }
    uint32_t w0 = cvt_scaled_pk4<CMX_FMT_E4M3>(c0[0], c0[1], scale), w1 = cvt_scaled_pk4<CMX_FMT_E4M3>(c0[2], c0[3], scale);
    uint32_t w2 = cvt_scaled_pk4<CMX_FMT_E4M3>(c1[0], c1[1], scale), w3 = cvt_scaled_pk4<CMX_FMT_E4M3>(c1[2], c1[3], scale);
    if (amax >= 0x7F80u) {                                  // Inf / NaN in the block (rare)
        patch_nonfinite_fp8<CMX_FMT_E4M3, false>(d0, w0, w1);
        patch_nonfinite_fp8<CMX_FMT_E4M3, false>(d1, w2, w3);
    }
    const uint32_t sbyte = (uint32_t)(e + 127) & 0xFFu;
    // scale bytes of blocks b .. b+3 (lanes l, l+2, l+4, l+6 of one 16-lane row) in the lane of the first
    uint32_t s4 = sbyte;
    if constexpr (VEC_SCALES) {
        s4 |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x102, 0xF, 0xF, true) << 8;     // row_shl:2
        s4 |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x104, 0xF, 0xF, true) << 16;    // row_shl:4
        s4 |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)sbyte, 0x106, 0xF, 0xF, true) << 24;    // row_shl:6
    }
    if (!live) return;
    const bool pad = (kb == nb - 1) && (nb & 1u);
    const uint4 codes = make_uint4(w0, w1, w2, w3);
    for (uint32_t r0 = 0; r0 < top_k; r0 += 8) {
        if (r0 > 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[j] = r0 + j < top_k ? src2sorted[(size_t)row * top_k + r0 + j] : -1;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (dst[j] < 0) continue;
            *reinterpret_cast<uint4*>(out_codes + (size_t)dst[j] * ld_out + col) = codes;
            uint8_t* s = out_scales + (size_t)dst[j] * ld_outs;
            if constexpr (VEC_SCALES) {
                if ((threadIdx.x & 7u) == 0) *reinterpret_cast<uint32_t*>(s + kb) = s4;
            } else if (h == 0) {
                s[kb] = (uint8_t)sbyte;
                if (pad) s[nb] = 127;
            }
        }
    }
}

// One workgroup per token: the same two-lanes-per-block arithmetic in passes of 128 blocks, but the token's scale
// bytes are collected in LDS and every destination gets them as one run of 16-byte stores covering `scale_run` bytes
// (the scale row, its padding column and zeros up to a multiple of 16, or up to the whole pitch): with a pitch of a
// whole number of 128-byte lines no line of the scale array is ever written in part.  k <= 32768.
__global__ __launch_bounds__(256) void quant_scatter_row_kernel(const uint16_t* __restrict__ x, uint32_t ld_x,
                                                                 const int32_t* __restrict__ src2sorted,
                                                                 uint8_t* __restrict__ out_codes, uint32_t ld_out,
                                                                 uint8_t* __restrict__ out_scales, uint32_t ld_outs, uint32_t top_k,
                                                                 uint32_t nb, uint32_t scale_run) {
    __shared__ __attribute__((aligned(16))) uint8_t s_scale[1024 + 16];
    const uint32_t row = blockIdx.x, h = threadIdx.x & 1u;
    const uint16_t* xrow = x + (size_t)row * ld_x;
    // zeros behind the scale bytes, 127 in the padding column of an odd count
    for (uint32_t i = nb + threadIdx.x; i < scale_run; i += 256) s_scale[i] = (i == nb && (nb & 1u)) ? 127 : 0;
    for (uint32_t r0 = 0; r0 < top_k; r0 += 8) {
        int32_t dst[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = r0 + j < top_k ? src2sorted[(size_t)row * top_k + r0 + j] : -1;
        for (uint32_t kb0 = 0; kb0 < nb; kb0 += 256) {                 // two passes of 128 blocks in flight together
            uint4 raw[2][2];
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const uint32_t kb = kb0 + it * 128 + (threadIdx.x >> 1);
                raw[it][0] = raw[it][1] = make_uint4(0, 0, 0, 0);
                if (kb < nb) {
                    raw[it][0] = *reinterpret_cast<const uint4*>(xrow + kb * 32 + h * 16);
                    raw[it][1] = *reinterpret_cast<const uint4*>(xrow + kb * 32 + h * 16 + 8);
                }
            }
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const uint32_t kb = kb0 + it * 128 + (threadIdx.x >> 1);
                const uint32_t d0[4] = {raw[it][0].x, raw[it][0].y, raw[it][0].z, raw[it][0].w};
                const uint32_t d1[4] = {raw[it][1].x, raw[it][1].y, raw[it][1].z, raw[it][1].w};
                uint32_t a0[4], a1[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    a0[i] = d0[i] & 0x7FFF7FFFu;
                    a1[i] = d1[i] & 0x7FFF7FFFu;
                }
                uint32_t m = pk_max_u16(pk_max_u16(pk_max_u16(a0[0], a0[1]), pk_max_u16(a0[2], a0[3])),
                                        pk_max_u16(pk_max_u16(a1[0], a1[1]), pk_max_u16(a1[2], a1[3])));
                m = pk_max_u16(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xF, 0xF, true));      // the block's other lane
                const uint32_t amax = max(m & 0xFFFFu, m >> 16);
                const int e = block_exp_from_bf16_amax(amax, kEmaxE4M3);
                const uint32_t lim = (((uint32_t)(e + kEmaxE4M3 + 127) << 7) | 0x60u) * 0x10001u;
                const float scale = __uint_as_float((uint32_t)(e + 127) << 23);
                uint32_t c0[4], c1[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    c0[i] = pk_min_u16(a0[i], lim) | (d0[i] & 0x80008000u);
                    c1[i] = pk_min_u16(a1[i], lim) | (d1[i] & 0x80008000u);
                }
                uint32_t w0 = cvt_scaled_pk4<CMX_FMT_E4M3>(c0[0], c0[1], scale), w1 = cvt_scaled_pk4<CMX_FMT_E4M3>(c0[2], c0[3], scale);
                uint32_t w2 = cvt_scaled_pk4<CMX_FMT_E4M3>(c1[0], c1[1], scale), w3 = cvt_scaled_pk4<CMX_FMT_E4M3>(c1[2], c1[3], scale);
                if (amax >= 0x7F80u) {                                  // Inf / NaN in the block (rare)
                    patch_nonfinite_fp8<CMX_FMT_E4M3, false>(d0, w0, w1);
                    patch_nonfinite_fp8<CMX_FMT_E4M3, false>(d1, w2, w3);
                }
                if (kb >= nb) continue;
                if (r0 == 0 && h == 0) s_scale[kb] = (uint8_t)(e + 127);
                const uint4 codes = make_uint4(w0, w1, w2, w3);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (dst[j] >= 0) *reinterpret_cast<uint4*>(out_codes + (size_t)dst[j] * ld_out + kb * 32 + h * 16) = codes;
            }
        }
        __syncthreads();                                                // the token's scale bytes are complete
        for (uint32_t c = threadIdx.x; c < 8 * (scale_run / 16); c += 256) {
            const uint32_t j = c / (scale_run / 16), q = c - j * (scale_run / 16);
            const int32_t d = j == 0 ? dst[0] : j == 1 ? dst[1] : j == 2 ? dst[2] : j == 3 ? dst[3] : j == 4 ? dst[4] : j == 5 ? dst[5] : j == 6 ? dst[6] : dst[7];
            if (d >= 0) *reinterpret_cast<uint4*>(out_scales + (size_t)d * ld_outs + q * 16) = *reinterpret_cast<const uint4*>(s_scale + q * 16);
        }
    }
}

// ---- weighted top-k combine -----------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_stream16(const void* p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store_stream16(void* p, uint4 v) {
    __builtin_nontemporal_store((u32x4){v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4*>(p));
}

// Rows of whole 16-byte vectors: one lane per (token, 8 hidden elements), items numbered token-major, so that
// every lane has the same amount of work whatever the hidden size.  A lane reads its token's eight row indices
// and weights (the same addresses across most of a wavefront: one transaction), issues the eight 16-byte gathers
// together and only then starts the arithmetic.
__global__ __launch_bounds__(256) void unpermute_vec_kernel(const uint16_t* __restrict__ y, uint32_t ld_y, uint32_t rows,
                                                             const int32_t* __restrict__ src2sorted,
                                                             const float* __restrict__ probs, uint16_t* __restrict__ out,
                                                             uint32_t ld_out, uint32_t nvec, uint32_t top_k,
                                                             uint32_t total_items) {
    const uint32_t item = blockIdx.x * 256 + threadIdx.x;
    if (item >= total_items) return;
    const uint32_t t = item / nvec, v = item - t * nvec;
    const int32_t* idx = src2sorted + (size_t)t * top_k;
    const float* wts = probs + (size_t)t * top_k;
    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
    for (uint32_t k0 = 0; k0 < top_k; k0 += 8) {
        int32_t r[8];
        float w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const bool in = k0 + j < top_k;
            r[j] = in ? idx[k0 + j] : -1;
            w[j] = in ? wts[k0 + j] : 0.0f;
        }
        uint4 raw[8];
        bool ok[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            ok[j] = r[j] >= 0 && (uint32_t)r[j] < rows;
            // every row is read exactly once: a streaming (non-temporal) load keeps it out of the way of the others
            // (measured: 183 us instead of 209 us at 8192 tokens x top-8 x 7168)
            raw[j] = ok[j] ? load_stream16(y + (size_t)r[j] * ld_y + v * 8) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (k0 + j >= top_k) break;
            const uint32_t dd[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // separate multiply and add (no fused multiply-add): Muls then Add in fp32, in k order; a row that is
                // out of range contributes an exact zero
                const float t0 = ok[j] ? __fmul_rn(__uint_as_float(dd[i] << 16), w[j]) : 0.0f;
                const float t1 = ok[j] ? __fmul_rn(__uint_as_float(dd[i] & 0xFFFF0000u), w[j]) : 0.0f;
                acc[2 * i] = (k0 + j) == 0 ? t0 : __fadd_rn(acc[2 * i], t0);
                acc[2 * i + 1] = (k0 + j) == 0 ? t1 : __fadd_rn(acc[2 * i + 1], t1);
            }
        }
    }
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16(acc[2 * i]) | (f32_to_bf16(acc[2 * i + 1]) << 16);
    store_stream16(out + (size_t)t * ld_out + v * 8, make_uint4(o[0], o[1], o[2], o[3]));
}

// Any hidden size (the ragged tail element by element): one workgroup per token; a lane owns 8 consecutive hidden
// elements per step.
template <int KMAX>
__global__ __launch_bounds__(256) void unpermute_kernel(const uint16_t* __restrict__ y, uint32_t ld_y, uint32_t rows,
                                                         const int32_t* __restrict__ src2sorted,
                                                         const float* __restrict__ probs, uint16_t* __restrict__ out,
                                                         uint32_t ld_out, uint32_t hidden, uint32_t top_k) {
    const uint32_t t = blockIdx.x;
    __shared__ int32_t s_idx[KMAX];
    __shared__ float s_w[KMAX];
    if (threadIdx.x < top_k) {
        s_idx[threadIdx.x] = src2sorted[(size_t)t * top_k + threadIdx.x];
        s_w[threadIdx.x] = probs[(size_t)t * top_k + threadIdx.x];
    }
    __syncthreads();
    const uint32_t nvec = hidden >> 3;
    for (uint32_t v = threadIdx.x; v < nvec; v += blockDim.x) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
        for (uint32_t k0 = 0; k0 < top_k; k0 += 8) {
            uint4 raw[8];
            bool ok[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t k = k0 + j;
                const int32_t r = k < top_k ? s_idx[k] : -1;
                ok[j] = r >= 0 && (uint32_t)r < rows;
                raw[j] = ok[j] ? *reinterpret_cast<const uint4*>(y + (size_t)r * ld_y + v * 8) : make_uint4(0, 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t k = k0 + j;
                if (k >= top_k) break;
                const float w = s_w[k];
                const uint32_t dd[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // separate multiply and add (no fused multiply-add): matches Muls then Add in fp32
                    float t0 = ok[j] ? __fmul_rn(__uint_as_float(dd[i] << 16), w) : 0.0f;
                    float t1 = ok[j] ? __fmul_rn(__uint_as_float(dd[i] & 0xFFFF0000u), w) : 0.0f;
                    acc[2 * i] = k == 0 ? t0 : __fadd_rn(acc[2 * i], t0);
                    acc[2 * i + 1] = k == 0 ? t1 : __fadd_rn(acc[2 * i + 1], t1);
                }
            }
        }
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = f32_to_bf16(acc[2 * i]) | (f32_to_bf16(acc[2 * i + 1]) << 16);
        *reinterpret_cast<uint4*>(out + (size_t)t * ld_out + v * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    }
    // ragged tail (hidden % 8 != 0)
    for (uint32_t c = (nvec << 3) + threadIdx.x; c < hidden; c += blockDim.x) {
        float acc = 0.0f;
        for (uint32_t k = 0; k < top_k; ++k) {
            const int32_t r = s_idx[k];
            const bool ok = r >= 0 && (uint32_t)r < rows;
            const float term = ok ? __fmul_rn(bf16_to_f32(y[(size_t)r * ld_y + c]), s_w[k]) : 0.0f;
            acc = k == 0 ? term : __fadd_rn(acc, term);
        }
        out[(size_t)t * ld_out + c] = (uint16_t)f32_to_bf16(acc);
    }
}

constexpr int kMaxTopK = 64;

__global__ void fill_i32_kernel(int32_t* p, uint32_t n, int32_t v) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---- per-token INT8 quantise + scatter -------------------------------------------------------------
// One workgroup per token: q = rint(x * 127 / rowmax) (round half to even), scale = rowmax / 127, the
// row written to each of its top_k destinations.  The row is read twice (maximum, then codes); the second
// read comes from the cache.  k % 8 == 0, rows 16-byte aligned.
__global__ __launch_bounds__(256) void int8_quant_scatter_kernel(const uint16_t* __restrict__ x, uint32_t ld_x,
                                                                 const int32_t* __restrict__ src2sorted,
                                                                 int8_t* __restrict__ codes, uint32_t ld_codes,
                                                                 float* __restrict__ scales, uint32_t k, uint32_t top_k) {
    __shared__ uint32_t wave_max[4];
    const uint32_t t = blockIdx.x;
    const uint16_t* row = x + (size_t)t * ld_x;
    const uint32_t chunks = k / 8;
    uint32_t m = 0;                                     // largest sign-cleared bf16 pattern == largest magnitude
    for (uint32_t c = threadIdx.x; c < chunks; c += 256) {
        const uint4 v = *reinterpret_cast<const uint4*>(row + 8 * c);
        m = pk_max_u16(m, v.x & 0x7FFF7FFFu);
        m = pk_max_u16(m, v.y & 0x7FFF7FFFu);
        m = pk_max_u16(m, v.z & 0x7FFF7FFFu);
        m = pk_max_u16(m, v.w & 0x7FFF7FFFu);
    }
    m = max(m & 0xFFFFu, m >> 16);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, d));
    if ((threadIdx.x & 63u) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    m = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
    const float rowmax = __uint_as_float(m << 16);
    const bool zero = !(rowmax > 0.0f);                 // an all-zero row: codes 0, scale 0
    const float div = zero ? 1.0f : rowmax;
    if (threadIdx.x < top_k) {
        const int32_t dst = src2sorted ? src2sorted[t * top_k + threadIdx.x] : (int32_t)t;
        if (dst >= 0) scales[dst] = __fdiv_rn(rowmax, 127.0f);
    }
    for (uint32_t c = threadIdx.x; c < chunks; c += 256) {
        const uint4 v = *reinterpret_cast<const uint4*>(row + 8 * c);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
        uint32_t out[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xv = __uint_as_float((i & 1) ? (d[i >> 1] & 0xFFFF0000u) : (d[i >> 1] << 16));
            const int q = zero ? 0 : (int)rintf(__fdiv_rn(__fmul_rn(xv, 127.0f), div));
            out[i >> 2] |= ((uint32_t)q & 0xFFu) << (8 * (i & 3));
        }
        for (uint32_t r = 0; r < top_k; ++r) {
            const int32_t dst = src2sorted ? src2sorted[t * top_k + r] : (int32_t)t;
            if (dst >= 0) *reinterpret_cast<uint2*>(codes + (size_t)dst * ld_codes + 8 * c) = make_uint2(out[0], out[1]);
        }
    }
}

}  // namespace
}  // namespace cmx

int cmx::preload_routing_kernels() {
    hipFuncAttributes attr;
    CMX_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(cmx::route_hist_kernel)));
    return CMX_OK;
}

extern "C" size_t cmx_moe_routing_workspace_bytes(uint32_t routes, uint32_t experts) {
    const size_t chunks = (routes + cmx::kChunk - 1) / cmx::kChunk;
    return cmx::round_up_sz((chunks ? chunks : 1) * (size_t)experts * sizeof(uint32_t), 256);
}

extern "C" int cmx_moe_init_routing(const int32_t* expert_idx, uint32_t tokens, uint32_t top_k, uint32_t experts,
                                    int32_t* sorted2src, int32_t* src2sorted, int32_t* counts, void* workspace,
                                    cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(expert_idx && sorted2src && src2sorted && counts && workspace, "null pointer");
    CMX_REQUIRE(experts > 0 && experts <= 8192, "experts must be in [1, 8192]");
    CMX_REQUIRE(top_k > 0, "top_k must be positive");
    CMX_REQUIRE((uint64_t)tokens * top_k < (1ull << 31), "too many routes");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t routes = tokens * top_k;
    const uint32_t chunks = ceil_div(routes, kChunk);
    uint32_t* hist = static_cast<uint32_t*>(workspace);
    if (routes == 0) {
        hipLaunchKernelGGL(fill_i32_kernel, dim3(ceil_div(experts, 256)), dim3(256), 0, s, counts, experts, 0);
        CMX_LAUNCH_CHECK();
        return CMX_OK;
    }
    uint32_t key_bits = 0;
    while ((1u << key_bits) < experts) ++key_bits;
    hipLaunchKernelGGL(route_hist_kernel, dim3(chunks), dim3(64), experts * sizeof(uint32_t), s, expert_idx, routes,
                       experts, hist);
    CMX_LAUNCH_CHECK();
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(1024), (experts + 1024) * sizeof(uint32_t), s, hist, chunks,
                       experts, counts);
    CMX_LAUNCH_CHECK();
    hipLaunchKernelGGL(route_scatter_kernel, dim3(chunks), dim3(64), experts * sizeof(uint32_t), s, expert_idx, routes,
                       experts, key_bits, hist, sorted2src, src2sorted);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

extern "C" uint32_t cmx_packed_row_bytes(uint32_t k) { return cmx::round_up(k + cmx::scale_cols(k), 32); }

extern "C" int cmx_quant_scatter(const void* x, uint32_t ld_x, const int32_t* src2sorted, uint8_t* out_codes,
                                 uint32_t ld_out, uint8_t* out_scales, uint32_t ld_outs, uint32_t tokens, uint32_t k,
                                 uint32_t top_k, cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(x && src2sorted && out_codes && out_scales, "null pointer");
    if (tokens == 0 || k == 0 || top_k == 0) return CMX_OK;
    CMX_REQUIRE(k % 32 == 0, "k must be a multiple of 32");
    CMX_REQUIRE(ld_x >= k && ld_x % 8 == 0 && aligned16(x), "input rows must be 16-byte aligned");
    CMX_REQUIRE(ld_out >= k && ld_out % 16 == 0 && aligned16(out_codes), "output rows must be 16-byte aligned");
    CMX_REQUIRE(ld_outs >= scale_cols(k), "scale pitch too small");
    const uint32_t nb = k / 32;
    CMX_REQUIRE((uint64_t)tokens * nb < (1ull << 32), "too many blocks for one launch");
    const uint32_t total = tokens * nb;
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Scale rows that can be written in 16-byte pieces take the row-wise kernel: the row, its padding column and zeros
    // up to a multiple of 16 bytes (never beyond: in the packed wire row, whose scale bytes sit behind the codes of the
    // same row, round_up(scale_cols, 16) <= round_up(scale_cols, 32) = the bytes the row has left behind its codes).
    // Only a scale array that is an allocation of its own -- one that does not overlap the code rows -- gets whole
    // pitches written when the pitch is the next multiple of 128, so that every 128-byte line of it is written whole.
    const uint32_t run16 = round_up(scale_cols(k), 16);
    if (ld_outs % 16 == 0 && aligned16(out_scales) && run16 <= ld_outs && nb <= 1024) {
        const uint64_t dst_rows = (uint64_t)tokens * top_k;
        const uintptr_t c0 = reinterpret_cast<uintptr_t>(out_codes), s0 = reinterpret_cast<uintptr_t>(out_scales);
        const bool disjoint = s0 >= c0 + dst_rows * ld_out || s0 + dst_rows * ld_outs <= c0;
        const uint32_t run = (disjoint && ld_outs == round_up(scale_cols(k), 128)) ? ld_outs : run16;
        hipLaunchKernelGGL(quant_scatter_row_kernel, dim3(tokens), dim3(256), 0, s, xp, ld_x, src2sorted, out_codes, ld_out,
                           out_scales, ld_outs, top_k, nb, run);
        CMX_LAUNCH_CHECK();
        return CMX_OK;
    }
    const bool vec_scales = nb % 4 == 0 && ld_outs % 4 == 0 && (reinterpret_cast<uintptr_t>(out_scales) & 3u) == 0;
    const dim3 grid(ceil_div(total, 128));
    if (vec_scales)
        hipLaunchKernelGGL((quant_scatter_kernel<true>), grid, dim3(256), 0, s, xp, ld_x, src2sorted, out_codes, ld_out,
                           out_scales, ld_outs, tokens, k, top_k, nb, total);
    else
        hipLaunchKernelGGL((quant_scatter_kernel<false>), grid, dim3(256), 0, s, xp, ld_x, src2sorted, out_codes, ld_out,
                           out_scales, ld_outs, tokens, k, top_k, nb, total);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

extern "C" int cmx_int8_quant_scatter(const void* x, uint32_t ld_x, const int32_t* src2sorted, int8_t* codes,
                                      uint32_t ld_codes, float* scales, uint32_t tokens, uint32_t k, uint32_t top_k,
                                      cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(x && codes && scales, "null pointer");
    if (tokens == 0 || k == 0) return CMX_OK;
    CMX_REQUIRE(top_k >= 1 && top_k <= 256, "top_k must be in [1, 256]");
    CMX_REQUIRE((uint64_t)tokens * top_k < (1ull << 32), "tokens * top_k must stay below 2^32");
    CMX_REQUIRE(src2sorted != nullptr || top_k == 1, "without a destination table every token has one destination");
    CMX_REQUIRE(k % 8 == 0, "k must be a multiple of 8");
    CMX_REQUIRE(ld_x >= k && ld_x % 8 == 0 && aligned16(x), "input rows must be 16-byte aligned");
    CMX_REQUIRE(ld_codes >= k && ld_codes % 8 == 0 && (reinterpret_cast<uintptr_t>(codes) & 7u) == 0,
                "output rows must be 8-byte aligned");
    hipLaunchKernelGGL(int8_quant_scatter_kernel, dim3(tokens), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(x), ld_x, src2sorted, codes, ld_codes, scales, k, top_k);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

extern "C" int cmx_moe_token_unpermute(const void* y, uint32_t ld_y, uint32_t rows, const int32_t* src2sorted,
                                       const float* probs, void* out, uint32_t ld_out, uint32_t tokens,
                                       uint32_t hidden, uint32_t top_k, cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(y && src2sorted && probs && out, "null pointer");
    if (tokens == 0 || hidden == 0) return CMX_OK;
    CMX_REQUIRE(top_k > 0 && top_k <= (uint32_t)kMaxTopK, "top_k must be in [1, 64]");
    CMX_REQUIRE(ld_y >= hidden && ld_out >= hidden, "row pitch smaller than a row");
    CMX_REQUIRE(ld_y % 8 == 0 && ld_out % 8 == 0 && aligned16(y) && aligned16(out), "rows must be 16-byte aligned");
    if (hidden % 8 == 0 && (uint64_t)tokens * (hidden / 8) < (1ull << 32)) {
        const uint32_t nvec = hidden / 8, total = tokens * nvec;
        hipLaunchKernelGGL(unpermute_vec_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(y), ld_y, rows, src2sorted, probs, static_cast<uint16_t*>(out),
                           ld_out, nvec, top_k, total);
    } else {
        hipLaunchKernelGGL((unpermute_kernel<kMaxTopK>), dim3(tokens), dim3(256), 0, static_cast<hipStream_t>(stream),
                           static_cast<const uint16_t*>(y), ld_y, rows, src2sorted, probs, static_cast<uint16_t*>(out),
                           ld_out, hidden, top_k);
    }
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}
