// Layout normalisation for MX operands stored with K as the slow axis.
//
// The matmul kernels want both operands K-contiguous: codes [rows, K] and scales [rows, K/32].  The
// reference's generators also write the other orientation (examples/ascend950_mxfp8_matmul_reduce_scatter/
// scripts/gen_data_mxfp8_mmrs.py:309-330 with trans_b = 0, the setting of the fp8_mx_allgather_matmul,
// mxfp8_matmul_alltoall and fp8_mx_alltoallv_grouped_matmul run scripts): codes [K, N] with N contiguous and
// scales [K/64, N, 2], i.e. for every pair of K blocks the two scale bytes of a column sit together.
// mx_to_k_major_kernel turns that into the K-contiguous form: a byte transpose of the codes and a
// transpose of 16-bit units of the scales, both pure data movement (HBM bound: every byte is read once and
// written once).
//
// One workgroup moves a 128 (K) x 128 (N) tile: dword loads along N (128-byte rows), a 4 x 4 byte transpose
// in registers with v_perm_b32, dwords of four consecutive K bytes staged in LDS, 16-byte stores along K
// (128-byte rows).
#include <hip/hip_runtime.h>

#include "catccos_mx.h"
#include "mx_common.h"

namespace cmx {
namespace {

constexpr int kLt = 128;                 // tile edge in bytes, both ways
constexpr int kLtPitch = kLt / 4 + 1;    // LDS row pitch in dwords
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// bytes (i, j) -> (j, i) of the 4 x 4 byte matrix whose rows are r0..r3; c[j] = {r0.j, r1.j, r2.j, r3.j}
__device__ __forceinline__ void transpose4x4(uint32_t r0, uint32_t r1, uint32_t r2, uint32_t r3, uint32_t (&c)[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u);   // r0.0 r1.0 r0.1 r1.1
    const uint32_t t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);   // r0.2 r1.2 r0.3 r1.3
    const uint32_t t2 = __builtin_amdgcn_perm(r3, r2, 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
    c[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    c[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

// grid: (ceil(n / 128), ceil(k / 128), batch)
__global__ __launch_bounds__(256) void mx_to_k_major_kernel(const uint8_t* __restrict__ src, uint32_t ld_src,
                                                            const uint8_t* __restrict__ src_scale,
                                                            uint8_t* __restrict__ dst, uint32_t ld_dst,
                                                            uint8_t* __restrict__ dst_scale, uint32_t ld_dst_scale,
                                                            uint32_t k, uint32_t n, uint64_t src_batch,
                                                            uint64_t dst_batch, uint64_t src_scale_batch,
                                                            uint64_t dst_scale_batch, int vec_in) {
    __shared__ uint32_t tile[kLt * kLtPitch];            // [n][k / 4]
    const uint32_t t = threadIdx.x;
    const uint32_t n0 = blockIdx.x * kLt, k0 = blockIdx.y * kLt;
    src += blockIdx.z * src_batch;
    dst += blockIdx.z * dst_batch;
    if (src_scale != nullptr) {
        src_scale += blockIdx.z * src_scale_batch;
        dst_scale += blockIdx.z * dst_scale_batch;
    }

    // load: thread -> column quad nq (4 bytes along N) and row quads kq, kq + 8, ...
    const uint32_t nq = t & 31u;
    const uint32_t ncol = n0 + 4 * nq;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t kq = (t >> 5) + 8 * i;
        uint32_t r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t kr = k0 + 4 * kq + j;
            r[j] = 0;
            if (kr < k) {
                const uint8_t* p = src + (size_t)kr * ld_src + ncol;
                if (vec_in && ncol + 4 <= n) {
                    r[j] = *reinterpret_cast<const uint32_t*>(p);
                } else {
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        if (ncol + b < n) r[j] |= (uint32_t)p[b] << (8 * b);
                }
            }
        }
        uint32_t c[4];
        transpose4x4(r[0], r[1], r[2], r[3], c);
#pragma unroll
        for (int j = 0; j < 4; ++j) tile[(4 * nq + j) * kLtPitch + kq] = c[j];
    }
    __syncthreads();

    // store: thread -> 16 bytes along K of row n0 + t / 8 + 32 i (k is a multiple of 64, so a piece is whole or absent)
    const uint32_t part = t & 7u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t nr = (t >> 3) + 32 * i;
        const uint32_t kc = k0 + 16 * part;
        if (n0 + nr < n && kc < k) {
            const uint32_t* q = tile + nr * kLtPitch + 4 * part;
            *reinterpret_cast<uint4*>(dst + (size_t)(n0 + nr) * ld_dst + kc) = make_uint4(q[0], q[1], q[2], q[3]);
        }
    }

    // scales: the tile spans the K-block pairs k0 / 64 and k0 / 64 + 1; [pair][n][2] -> [n][2 pair + {0, 1}]
    if (src_scale != nullptr && t < (uint32_t)kLt && n0 + t < n) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t pair = k0 / 64 + h;
            if (pair * 64 < k) {
                const uint8_t* sp = src_scale + ((size_t)pair * n + n0 + t) * 2;
                uint8_t* dp = dst_scale + (size_t)(n0 + t) * ld_dst_scale + 2 * pair;
                dp[0] = sp[0];
                dp[1] = sp[1];
            }
        }
    }
}

// The same tile with 16-byte loads, for sources whose rows are 16-byte aligned and whose n is a multiple of 16 (a
// 16-byte piece is then whole or absent): a thread loads 16 bytes of four consecutive K rows (all four loads in flight
// before the first use), transposes its four 4 x 4 byte blocks and stages sixteen dwords.  The LDS tile is
// [n][32 dwords of K] with the dword index XORed by 4 (n / 16): the sixteen lanes-times-rows that write at once differ
// in n / 16 and in the low K bits and so hit 32 different banks, and the 16-byte runs the store phase reads stay whole.
// Every byte is touched once, so loads and stores are non-temporal (3 % on 485 MB of weights).
__global__ __launch_bounds__(256) void mx_to_k_major16_kernel(const uint8_t* __restrict__ src, uint32_t ld_src,
                                                              const uint8_t* __restrict__ src_scale,
                                                              uint8_t* __restrict__ dst, uint32_t ld_dst,
                                                              uint8_t* __restrict__ dst_scale, uint32_t ld_dst_scale,
                                                              uint32_t k, uint32_t n, uint64_t src_batch,
                                                              uint64_t dst_batch, uint64_t src_scale_batch,
                                                              uint64_t dst_scale_batch) {
    __shared__ __attribute__((aligned(16))) uint32_t tile[kLt * 32];   // [n][(k / 4) ^ swizzle(n)]
    const uint32_t t = threadIdx.x;
    const uint32_t n0 = blockIdx.x * kLt, k0 = blockIdx.y * kLt;
    src += blockIdx.z * src_batch;
    dst += blockIdx.z * dst_batch;

    // scales first (their loads overlap the tile's): [pair][n][2] -> [n][2 pair + {0, 1}], one 16-bit unit per thread
    uint32_t sval = 0;
    const uint32_t s_n = n0 + (t & 127u), s_pair = k0 / 64 + (t >> 7);
    const bool s_on = src_scale != nullptr && s_n < n && s_pair * 64 < k;
    if (s_on)
        sval = *reinterpret_cast<const uint16_t*>(src_scale + blockIdx.z * src_scale_batch + ((size_t)s_pair * n + s_n) * 2);

    const uint32_t nq = t & 7u, kq = t >> 3;          // 16 bytes along N, rows 4 kq .. 4 kq + 3
    const uint32_t ncol = n0 + 16 * nq;
    u32x4 r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t kr = k0 + 4 * kq + j;
        r[j] = u32x4{0, 0, 0, 0};
        if (kr < k && ncol < n) r[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (size_t)kr * ld_src + ncol));
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        uint32_t c[4];
        transpose4x4(r[0][d], r[1][d], r[2][d], r[3][d], c);
#pragma unroll
        for (int j = 0; j < 4; ++j) tile[(16 * nq + 4 * d + j) * 32 + (kq ^ (4 * nq))] = c[j];
    }
    __syncthreads();

    const uint32_t part = t & 7u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t nr = (t >> 3) + 32 * i;
        const uint32_t kc = k0 + 16 * part;
        if (n0 + nr < n && kc < k) {
            const u32x4 q = *reinterpret_cast<const u32x4*>(tile + nr * 32 + ((4 * part) ^ (4 * (nr >> 4))));
            __builtin_nontemporal_store(q, reinterpret_cast<u32x4*>(dst + (size_t)(n0 + nr) * ld_dst + kc));
        }
    }
    if (s_on)
        *reinterpret_cast<uint16_t*>(dst_scale + blockIdx.z * dst_scale_batch + (size_t)s_n * ld_dst_scale + 2 * s_pair) =
            (uint16_t)sval;
}

// FP4: two codes share a byte along the contiguous axis, so the same change of orientation is a transpose of 4-bit
// units: source [K, N/2] bytes (N pairs per byte, even column in the low nibble) -> destination [N, K/2] bytes (K pairs
// per byte).  A thread transposes an 8 x 8 block of nibbles held in eight dwords with the three-level masked-swap
// network (4-, 8- and 16-bit fields); a workgroup moves 128 (K) x 128 (N) codes.
__device__ __forceinline__ void transpose8x8_nibbles(uint32_t (&w)[8]) {
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
        const uint32_t t = ((w[i] >> 4) ^ w[i + 1]) & 0x0F0F0F0Fu;
        w[i + 1] ^= t;
        w[i] ^= t << 4;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (i & 2) continue;
        const uint32_t t = ((w[i] >> 8) ^ w[i + 2]) & 0x00FF00FFu;
        w[i + 2] ^= t;
        w[i] ^= t << 8;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t t = ((w[i] >> 16) ^ w[i + 4]) & 0x0000FFFFu;
        w[i + 4] ^= t;
        w[i] ^= t << 16;
    }
}

// grid: (ceil(n / 128), ceil(k / 128), batch); ld_src / ld_dst in bytes
__global__ __launch_bounds__(256) void mxfp4_to_k_major_kernel(const uint8_t* __restrict__ src, uint32_t ld_src,
                                                               const uint8_t* __restrict__ src_scale,
                                                               uint8_t* __restrict__ dst, uint32_t ld_dst,
                                                               uint8_t* __restrict__ dst_scale, uint32_t ld_dst_scale,
                                                               uint32_t k, uint32_t n, uint64_t src_batch,
                                                               uint64_t dst_batch, uint64_t src_scale_batch,
                                                               uint64_t dst_scale_batch, int vec_in) {
    constexpr int kPitch = 16 + 1;                       // dwords per staged destination row (128 K codes = 64 bytes)
    __shared__ uint32_t tile[kLt * kPitch];              // [n][k / 8]
    const uint32_t t = threadIdx.x;
    const uint32_t n0 = blockIdx.x * kLt, k0 = blockIdx.y * kLt;
    src += blockIdx.z * src_batch;
    dst += blockIdx.z * dst_batch;
    src_scale += blockIdx.z * src_scale_batch;
    dst_scale += blockIdx.z * dst_scale_batch;
    const uint32_t src_row_bytes = (n + 1) / 2;

    // load: thread -> 8 K rows (kb) x 8 N codes (nb): one dword of each row
    const uint32_t nb = t & 15u, kb = t >> 4;
    const uint32_t byte0 = n0 / 2 + 4 * nb;
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t kr = k0 + 8 * kb + j;
        w[j] = 0;
        if (kr < k) {
            const uint8_t* p = src + (size_t)kr * ld_src + byte0;
            if (vec_in && byte0 + 4 <= src_row_bytes) {
                w[j] = *reinterpret_cast<const uint32_t*>(p);
            } else {
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    if (byte0 + b < src_row_bytes) w[j] |= (uint32_t)p[b] << (8 * b);
            }
        }
    }
    transpose8x8_nibbles(w);                             // w[i] = codes k0 + 8 kb .. + 7 of column n0 + 8 nb + i
#pragma unroll
    for (int i = 0; i < 8; ++i) tile[(8 * nb + i) * kPitch + kb] = w[i];
    __syncthreads();

    // store: thread -> 16 bytes (32 K codes) of row n0 + t / 4 + 64 i; k is a multiple of 64, so a piece is whole or absent
    const uint32_t part = t & 3u;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t nr = (t >> 2) + 64 * i;
        const uint32_t kc = k0 + 32 * part;
        if (n0 + nr < n && kc < k) {
            const uint32_t* q = tile + nr * kPitch + 4 * part;
            *reinterpret_cast<uint4*>(dst + (size_t)(n0 + nr) * ld_dst + kc / 2) = make_uint4(q[0], q[1], q[2], q[3]);
        }
    }

    // scales: as for the 8-bit formats
    if (t < (uint32_t)kLt && n0 + t < n) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t pair = k0 / 64 + h;
            if (pair * 64 < k) {
                const uint8_t* sp = src_scale + ((size_t)pair * n + n0 + t) * 2;
                uint8_t* dp = dst_scale + (size_t)(n0 + t) * ld_dst_scale + 2 * pair;
                dp[0] = sp[0];
                dp[1] = sp[1];
            }
        }
    }
}

int fp4_to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst, uint32_t ld_dst,
                   uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n, uint32_t batch, hipStream_t s) {
    CMX_REQUIRE(src && src_scale && dst && dst_scale, "null pointer");
    CMX_REQUIRE(k > 0 && k % 64 == 0, "k must be a positive multiple of 64 (scale bytes come in pairs of K blocks)");
    CMX_REQUIRE(ld_src >= (n + 1) / 2 && ld_dst >= k / 2 && ld_dst_scale >= k / 32, "row pitch smaller than a row");
    CMX_REQUIRE(ld_dst % 16 == 0 && aligned16(dst), "destination rows must be 16-byte aligned");
    if (n == 0 || batch == 0) return CMX_OK;
    CMX_REQUIRE(batch <= 65535u && ceil_div(k, kLt) <= 65535u, "too many tiles for one launch");
    const int vec_in = ld_src % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 3u) == 0;
    dim3 grid(ceil_div(n, kLt), ceil_div(k, kLt), batch);
    hipLaunchKernelGGL(mxfp4_to_k_major_kernel, grid, dim3(256), 0, s, src, ld_src, src_scale, dst, ld_dst, dst_scale,
                       ld_dst_scale, k, n, (uint64_t)k * ld_src, (uint64_t)n * ld_dst, (uint64_t)(k / 32) * n,
                       (uint64_t)n * ld_dst_scale, vec_in);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

int to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst, uint32_t ld_dst,
               uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n, uint32_t batch, hipStream_t s) {
    CMX_REQUIRE(src && dst && (src_scale == nullptr) == (dst_scale == nullptr), "null pointer");
    CMX_REQUIRE(k > 0 && k % 64 == 0, "k must be a positive multiple of 64 (scale bytes come in pairs of K blocks)");
    CMX_REQUIRE(ld_src >= n && ld_dst >= k && (dst_scale == nullptr || ld_dst_scale >= k / 32), "row pitch smaller than a row");
    CMX_REQUIRE(ld_dst % 16 == 0 && aligned16(dst), "destination rows must be 16-byte aligned");
    if (n == 0 || batch == 0) return CMX_OK;
    CMX_REQUIRE(batch <= 65535u && ceil_div(k, kLt) <= 65535u, "too many tiles for one launch");
    const int vec_in = ld_src % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 3u) == 0;
    dim3 grid(ceil_div(n, kLt), ceil_div(k, kLt), batch);
    const bool scales16 = src_scale == nullptr || (((reinterpret_cast<uintptr_t>(src_scale) | reinterpret_cast<uintptr_t>(dst_scale)) & 1u) == 0 &&
                                                   ld_dst_scale % 2 == 0);
    if (ld_src % 16 == 0 && aligned16(src) && n % 16 == 0 && scales16) {
        hipLaunchKernelGGL(mx_to_k_major16_kernel, grid, dim3(256), 0, s, src, ld_src, src_scale, dst, ld_dst, dst_scale,
                           ld_dst_scale, k, n, (uint64_t)k * ld_src, (uint64_t)n * ld_dst, (uint64_t)(k / 32) * n,
                           (uint64_t)n * ld_dst_scale);
        CMX_LAUNCH_CHECK();
        return CMX_OK;
    }
    hipLaunchKernelGGL(mx_to_k_major_kernel, grid, dim3(256), 0, s, src, ld_src, src_scale, dst, ld_dst, dst_scale,
                       ld_dst_scale, k, n, (uint64_t)k * ld_src, (uint64_t)n * ld_dst, (uint64_t)(k / 32) * n,
                       (uint64_t)n * ld_dst_scale, vec_in);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

// workspace carve-up of the *_ex entry points: normalised A (when stored [K, M]) then normalised B (when stored [K, N])
struct ExLayout {
    size_t a_codes, a_scales, b_codes, b_scales, total;
};

ExLayout ex_layout(uint64_t a_rows, uint64_t b_rows, uint32_t k, int trans_a, int b_k_major, int fmt = CMX_FMT_E4M3) {
    const uint32_t kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k;
    ExLayout L{};
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off += round_up_sz(bytes, 256);
        return at;
    };
    if (trans_a) {
        L.a_codes = take(a_rows * kbytes);
        L.a_scales = take(a_rows * (k / 32));
    }
    if (!b_k_major) {
        L.b_codes = take(b_rows * kbytes);
        L.b_scales = take(b_rows * (k / 32));
    }
    L.total = off;
    return L;
}

bool fmt_is_8bit(int fmt) { return fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2; }
bool fmt_has_layouts(int fmt) { return fmt_is_8bit(fmt) || fmt == CMX_FMT_E2M1; }

// operand [k, rows] in the format's K-slow storage -> K-contiguous, packed pitches
int normalise(const uint8_t* src, const uint8_t* src_scale, uint8_t* dst, uint8_t* dst_scale, uint32_t k, uint32_t rows,
              uint32_t batch, int fmt, hipStream_t s) {
    if (fmt == CMX_FMT_E2M1)
        return fp4_to_k_major(src, (rows + 1) / 2, src_scale, dst, k / 2, dst_scale, k / 32, k, rows, batch, s);
    return to_k_major(src, rows, src_scale, dst, k, dst_scale, k / 32, k, rows, batch, s);
}

}  // namespace
}  // namespace cmx

int cmx::preload_layout_kernels() {
    hipFuncAttributes attr;
    CMX_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(cmx::mx_to_k_major16_kernel)));
    return CMX_OK;
}

extern "C" int cmx_mx_to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst,
                                 uint32_t ld_dst, uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n,
                                 uint32_t batch, cmx_stream_t stream) {
    if (!src_scale || !dst_scale) {
        cmx::set_error("null pointer");
        return CMX_EINVAL;
    }
    return cmx::to_k_major(src, ld_src, src_scale, dst, ld_dst, dst_scale, ld_dst_scale, k, n, batch,
                           static_cast<hipStream_t>(stream));
}

extern "C" int cmx_mxfp4_to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst,
                                    uint32_t ld_dst, uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n,
                                    uint32_t batch, cmx_stream_t stream) {
    return cmx::fp4_to_k_major(src, ld_src, src_scale, dst, ld_dst, dst_scale, ld_dst_scale, k, n, batch,
                               static_cast<hipStream_t>(stream));
}

// the code part alone (INT8 weights stored [batch, k, n] -> [batch, n, k])
extern "C" int cmx_bytes_to_k_major(const uint8_t* src, uint32_t ld_src, uint8_t* dst, uint32_t ld_dst, uint32_t k, uint32_t n,
                                    uint32_t batch, cmx_stream_t stream) {
    return cmx::to_k_major(src, ld_src, nullptr, dst, ld_dst, nullptr, 0, k, n, batch, static_cast<hipStream_t>(stream));
}

extern "C" size_t cmx_mx_gemm_ex_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int trans_a, int trans_b) {
    return cmx::ex_layout(m, n, k, trans_a, trans_b).total;
}

extern "C" int cmx_mx_gemm_ex(const uint8_t* a, const uint8_t* a_scale, const uint8_t* b, const uint8_t* b_scale, void* c,
                              uint32_t ldc, uint32_t m, uint32_t n, uint32_t k, int fmt, int out_type, int trans_a,
                              int trans_b, void* workspace, cmx_stream_t stream) {
    using namespace cmx;
    if (m == 0 || n == 0) return CMX_OK;
    CMX_REQUIRE(fmt_has_layouts(fmt), "unknown element format");
    CMX_REQUIRE(k > 0 && k % 64 == 0, "k must be a positive multiple of 64");
    const ExLayout L = ex_layout(m, n, k, trans_a, trans_b, fmt);
    CMX_REQUIRE(L.total == 0 || (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0),
                "workspace missing or not 256-byte aligned");
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k;
    if (trans_a) {
        int rc = normalise(a, a_scale, ws + L.a_codes, ws + L.a_scales, k, m, 1, fmt, s);
        if (rc != CMX_OK) return rc;
        a = ws + L.a_codes;
        a_scale = ws + L.a_scales;
    }
    if (!trans_b) {
        int rc = normalise(b, b_scale, ws + L.b_codes, ws + L.b_scales, k, n, 1, fmt, s);
        if (rc != CMX_OK) return rc;
        b = ws + L.b_codes;
        b_scale = ws + L.b_scales;
    }
    return cmx_mx_gemm(a, kbytes, a_scale, k / 32, b, kbytes, b_scale, k / 32, c, ldc, m, n, k, fmt, out_type, stream);
}

extern "C" size_t cmx_mx_gmm_ex_workspace_bytes(uint32_t groups, uint32_t n, uint32_t k, int trans_b) {
    const size_t meta = cmx::round_up_sz(cmx_mx_gmm_workspace_bytes(groups), 256);
    return meta + cmx::ex_layout(0, (uint64_t)groups * n, k, 0, trans_b).total;
}

extern "C" int cmx_mx_gmm_ex(const uint8_t* a, const uint8_t* a_scale, const uint8_t* b, const uint8_t* b_scale, void* c,
                             uint32_t ldc, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n,
                             uint32_t k, int fmt, int out_type, int trans_b, void* workspace, cmx_stream_t stream) {
    using namespace cmx;
    if (m_total == 0 || n == 0) return CMX_OK;
    CMX_REQUIRE(fmt_has_layouts(fmt), "unknown element format");
    CMX_REQUIRE(k > 0 && k % 64 == 0, "k must be a positive multiple of 64");
    CMX_REQUIRE(groups > 0 && workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
                "workspace missing or not 256-byte aligned");
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const size_t meta = round_up_sz(cmx_mx_gmm_workspace_bytes(groups), 256);
    if (!trans_b) {
        CMX_REQUIRE(fmt != CMX_FMT_E2M1 || n % 2 == 0, "FP4 weights stored [groups, k, n / 2] need an even n");
        const ExLayout L = ex_layout(0, (uint64_t)groups * n, k, 0, 0, fmt);
        int rc = normalise(b, b_scale, ws + meta + L.b_codes, ws + meta + L.b_scales, k, n, groups, fmt,
                           static_cast<hipStream_t>(stream));
        if (rc != CMX_OK) return rc;
        b = ws + meta + L.b_codes;
        b_scale = ws + meta + L.b_scales;
    }
    const uint32_t kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k;
    return cmx_mx_gmm(a, kbytes, a_scale, k / 32, b, b_scale, c, ldc, group_sizes, groups, m_total, n, k, fmt, out_type, ws, stream);
}

// ---- pre-tiled weights -------------------------------------------------------------------------------------------
// The weights-to-registers grouped kernel reads the weights of a 256-row tile slab by slab (128 bytes of K), and within
// a slab every wavefront reads its own 8 KiB as eight loads of 1 KiB: [group][tile][slab][wavefront 0..3][step h]
// [fragment f][register half][lane / 32][lane % 32][16 bytes].  The piece at (h, f, half, lh, l32) is bytes
// 128 slab + 64 h + 32 half + 16 lh .. + 16 of the tile row that lane l32 feeds to the MFMA as weight fragment f:
//   plain tiles    row 256 tile + 64 wavefront + 32 f + l32
//   gate|up tiles  row 128 tile + 32 wavefront + l32 of the gate half (f = 0) or of the up half (f = 1)
// (rows past the end repeat the last one, as the kernels' own clamped reads do).
namespace cmx {
namespace {
constexpr uint32_t kPretileRows = 256;

__global__ __launch_bounds__(512) void mx_pretile_weights_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                                 uint32_t n, uint32_t kbytes, uint32_t w_tiles, int pair) {
    // one workgroup: the 512 pieces of one (group, tile, slab, wavefront) -- 64 rows x 128 bytes, read as whole lines
    const uint32_t t = threadIdx.x;
    const uint32_t l32 = t & 31u, lh = (t >> 5) & 1u, half = (t >> 6) & 1u, f = (t >> 7) & 1u, h = t >> 8;
    const uint32_t nslab = kbytes / 128;
    const uint32_t ww = blockIdx.x & 3u;
    const uint32_t slab = (blockIdx.x >> 2) % nslab;
    const uint32_t tile = (blockIdx.x >> 2) / nslab;          // tile of the group
    const uint32_t g = blockIdx.y;
    uint32_t row;
    if (pair) {
        const uint32_t hn = n >> 1;
        uint32_t r = tile * (kPretileRows / 2) + ww * 32 + l32;
        r = r < hn ? r : hn - 1;
        row = f ? hn + r : r;
    } else {
        row = tile * kPretileRows + ww * 64 + f * 32 + l32;
        row = row < n ? row : n - 1;
    }
    const uint32_t col = slab * 128 + h * 64 + half * 32 + lh * 16;
    const uint4 v = *reinterpret_cast<const uint4*>(src + ((size_t)g * n + row) * kbytes + col);
    const size_t piece = (((size_t)g * w_tiles + tile) * nslab + slab) * 2048 + ww * 512 + t;
    *reinterpret_cast<uint4*>(dst + piece * 16) = v;
}

uint32_t pretile_tiles(uint32_t n, int pair) { return pair ? ceil_div(n / 2, kPretileRows / 2) : ceil_div(n, kPretileRows); }
}  // namespace
}  // namespace cmx

extern "C" size_t cmx_mx_pretiled_weight_bytes(uint32_t groups, uint32_t n, uint32_t k, int pair_gate_up) {
    if (groups == 0 || n == 0 || k == 0 || k % 512 != 0 || (pair_gate_up && n % 64 != 0)) return 0;
    return (size_t)groups * cmx::pretile_tiles(n, pair_gate_up) * cmx::kPretileRows * k;
}

extern "C" int cmx_mx_pretile_weights(const uint8_t* b, uint8_t* out, uint32_t groups, uint32_t n, uint32_t k,
                                      int pair_gate_up, cmx_stream_t stream) {
    using namespace cmx;
    if (groups == 0 || n == 0) return CMX_OK;
    CMX_REQUIRE(b && out, "null pointer");
    CMX_REQUIRE(k > 0 && k % 512 == 0, "k must be a positive multiple of 512");
    CMX_REQUIRE(!pair_gate_up || n % 64 == 0, "gate|up weights need n to be a multiple of 64");
    CMX_REQUIRE(aligned16(b) && aligned16(out), "weights must be 16-byte aligned");
    CMX_REQUIRE(groups <= 65535, "at most 65535 groups");
    const uint32_t w_tiles = pretile_tiles(n, pair_gate_up);
    const uint64_t blocks = (uint64_t)w_tiles * (k / 128) * 4;
    CMX_REQUIRE(blocks < (1ull << 31), "weight matrix too large");
    hipLaunchKernelGGL(mx_pretile_weights_kernel, dim3((uint32_t)blocks, groups), dim3(512), 0, static_cast<hipStream_t>(stream), b,
                       out, n, k, w_tiles, pair_gate_up ? 1 : 0);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}
