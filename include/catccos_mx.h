/*
 * catccos_mx.h - C ABI of the MI355X (gfx950) MX compute core.
 *
 * Plain C: pointers are device pointers unless a parameter is named host_*, sizes are in
 * elements unless a name ends in _bytes.  Every entry point is asynchronous on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream) and returns 0 on success or a
 * negative CMX_E* code; cmx_last_error() returns a thread-local message for the last
 * failure.  Nothing here allocates device memory except the cmx_rt_* runtime shim.
 *
 * Each group names the reference interface it replaces (paths relative to the reference
 * checkout).
 */
#ifndef CATCCOS_MX_H
#define CATCCOS_MX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CMX_OK 0
#define CMX_EINVAL (-1)   /* bad argument (shape, alignment, null pointer) */
#define CMX_ERUNTIME (-2) /* HIP runtime reported an error               */
#define CMX_ENOSPACE (-3) /* workspace too small                         */

/* element formats (E8M0 block-32 scales in every case) */
#define CMX_FMT_E4M3 0
#define CMX_FMT_E5M2 1
#define CMX_FMT_E2M1 2 /* FP4, two codes per byte, even column in the low nibble */
#define CMX_FMT_E1M2 3 /* FP4 with values k/4, k = 0..7 (quantizer and dequantizer only), packed like E2M1 */

/* rounding of the element cast */
#define CMX_ROUND_RNE 0 /* IEEE nearest-even: runtime activations            */
#define CMX_ROUND_LUT 1 /* nearest table value, tie -> smaller magnitude, -0 -> +0: offline weights, FP4 golden */

/* output types of the matmul entry points */
#define CMX_OUT_BF16 0
#define CMX_OUT_FP16 1
#define CMX_OUT_FP32 2

typedef void* cmx_stream_t;

int cmx_version(void);
const char* cmx_last_error(void);

/* One-time set-up on the current device (no counterpart in the reference, whose kernels need none): raises the
 * dynamic-LDS limit of every matmul kernel, reads the CU count and resolves the static schedule array of
 * cmx_mx_gmm_swiglu_quant_noalloc.  Optional -- every entry point does what it needs on first use -- but a caller
 * that captures streams into graphs must call it first: raising a kernel's LDS limit is not allowed during capture. */
int cmx_init(void);

/* ------------------------------------------------------------------------------------------
 * Runtime shim: what the host plugin layer needs from the device runtime.
 * Replaces aclrtMalloc / aclrtFree / aclrtMallocHost / aclrtFreeHost / aclrtMemcpy /
 * aclrtMemset / aclrtSynchronizeStream as used by utils/info.h:134-214 and every
 * examples/<op>/<op>_host.h AllocateDeviceSpace / WriteResultFile.
 * ---------------------------------------------------------------------------------------- */
int cmx_rt_device_count(int* count);
int cmx_rt_set_device(int device);
int cmx_rt_malloc(void** ptr, size_t bytes);
int cmx_rt_free(void* ptr);
int cmx_rt_malloc_host(void** ptr, size_t bytes);
int cmx_rt_free_host(void* ptr);
int cmx_rt_memcpy_h2d(void* dst, const void* host_src, size_t bytes);
int cmx_rt_memcpy_d2h(void* host_dst, const void* src, size_t bytes);
int cmx_rt_memset(void* dst, int value, size_t bytes);
int cmx_rt_stream_create(cmx_stream_t* stream);
int cmx_rt_stream_destroy(cmx_stream_t stream);
int cmx_rt_stream_sync(cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * MX block quantizer.
 * Replaces CommBlockMxQuant::operator() / ComputeMxQuant
 * (include/catccos/comm/block/comm_block_mx_quant.hpp:154-316, 412-664) launched by
 * MxQuantAllGather<<<>>> (examples/ascend950_mx_quant_allgather/mx_quant_allgather_device.h:108-141);
 * results follow the golden _quantize_axis_last_fp8 / _quantize_axis_last
 * (examples/utils/gen_mx_quant_allgather_data.py:255-313, 414-449).
 *
 *   x       bf16 [rows, cols], row pitch ld_x elements
 *   codes   u8   [rows, cols] (FP4: [rows, ceil(cols/2)]), row pitch ld_codes bytes
 *   scales  u8   [rows, RoundUp2(ceil(cols/32))], row pitch ld_scales bytes; padding column = 127.
 *           A pitch of exactly ceil(cols/32) selects unpadded scale rows (the [M, N/32] file of
 *           examples/ascend950_mx_quant_allgather/mx_quant_allgather_host.h:47-87): no padding column is written.
 *
 * Non-finite input follows the golden, not the reference device (which writes scale 0xFF and NaN codes for such
 * a block, comm_block_mx_quant.hpp:496-515).  A block whose maximum is Inf or NaN: 8-bit formats take the
 * exponent field as it is (scale byte 247 for E4M3, 240 for E5M2) and scale the finite elements by it, +-Inf
 * becomes the largest code with its sign, NaN the NaN code 0x7F | sign (CMX_ROUND_RNE) or code 0
 * (CMX_ROUND_LUT).  4-bit formats: an Inf maximum gives scale byte 254 and +-Inf the largest code; a NaN
 * maximum gives scale byte 255 and code 0 for every element of the block.
 * ---------------------------------------------------------------------------------------- */
int cmx_mx_quant(const void* x, uint32_t ld_x, uint8_t* codes, uint32_t ld_codes, uint8_t* scales,
                 uint32_t ld_scales, uint32_t rows, uint32_t cols, int fmt, int round_mode, cmx_stream_t stream);

/* Dequantize (test/debug helper, same layouts): out fp32 [rows, cols]. */
int cmx_mx_dequant(const uint8_t* codes, uint32_t ld_codes, const uint8_t* scales, uint32_t ld_scales, float* out,
                   uint32_t ld_out, uint32_t rows, uint32_t cols, int fmt, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Dense MX matmul  C[m,n] = sum_k deq(A)[m,k] * deq(B)[n,k]   (both operands K-contiguous).
 * Replaces the AIC loop of MatmulReduceScatterMxTla
 * (include/catccos/dgemm/kernel/matmul_reduce_scatter_mx_tla.hpp:190-315: blockMmad(A,B,C,shape,
 * scaleA,scaleB)) for one device's full M x N x K product; golden
 * examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/gen_data_mxfp8_mmrs.py:343-355.
 *
 *   a  codes [m, k] (FP4: k/2 bytes), pitch lda bytes;  a_scale u8 [m, k/32], pitch ld_as bytes
 *   b  codes [n, k] (transposed weight), pitch ldb;     b_scale u8 [n, k/32], pitch ld_bs
 *   c  [m, n] of out_type, pitch ldc elements
 * k must be a multiple of 32; operand rows 16-byte aligned.
 * ---------------------------------------------------------------------------------------- */
int cmx_mx_gemm(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b,
                uint32_t ldb, const uint8_t* b_scale, uint32_t ld_bs, void* c, uint32_t ldc, uint32_t m,
                uint32_t n, uint32_t k, int fmt, int out_type, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Grouped MX matmul over ragged expert groups.
 * Replaces the AIC tile loops of Ascend950GmmAllToAllKernel
 * (include/catccos/dgemm/kernel/ascend950_gmm_alltoall.hpp:219-324) and
 * MxAllToAllVGroupedMatmulTla (include/catccos/dgemm/kernel/mx_alltoallv_group_matmul.hpp),
 * including their per-expert offset arithmetic (ascend950_alltoall_gmm.hpp:238-322).
 *
 *   group_sizes  int32 [groups] ON DEVICE (rows per expert, in order; zeros allowed)
 *   a / a_scale  rows of all groups back to back, m_total = sum(group_sizes) rows
 *   b / b_scale  [groups, n, k] / [groups, n, RoundUp2(k/32)], dense (scale rows padded to an even count, as the
 *                quantizer and the reference's generators write them; no padding when k is a multiple of 64)
 *   c            [m_total, n]
 *   workspace    >= cmx_mx_gmm_workspace_bytes(groups) bytes (tile schedule metadata)
 * Rows beyond sum(group_sizes) (up to m_total) are left untouched.
 * ---------------------------------------------------------------------------------------- */
size_t cmx_mx_gmm_workspace_bytes(uint32_t groups);
int cmx_mx_gmm(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b,
               const uint8_t* b_scale, void* c, uint32_t ldc, const int32_t* group_sizes, uint32_t groups,
               uint32_t m_total, uint32_t n, uint32_t k, int fmt, int out_type, void* workspace,
               cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Grouped MXFP8 matmul with fused SwiGLU and MX requant (GMM1 of the FFN).
 * Replaces Ascend950AllToAllGmmKernel's AIC loop (ascend950_alltoall_gmm.hpp:193-323: gate and
 * up products per tile) + SwigluBf16RegBaseVf
 * (include/catccos/epilogue/block/block_epilogue_regbase_swiglu.hpp:38-78) +
 * Ascend950SwigluMxQuantFromUbKernel::ComputeUbTile
 * (examples/aux_ops/ascend950_swiglu_from_ub.h:333-373); golden gen_data_moe.py:646-658.
 *
 *   b / b_scale   [groups, n, k]: rows [0, n/2) = gate (gets SiLU), rows [n/2, n) = up
 *   act_codes     u8 E4M3 [m_total, n/2], pitch ld_act bytes
 *   act_scales    u8 E8M0 [m_total, RoundUp2(n/64)], pitch ld_acts bytes
 *   act_bf16      optional (may be NULL): bf16 [m_total, n/2] SwiGLU output before requant
 * n must be a multiple of 64.  h = bf16(A.B) and act = bf16(silu(gate)*up) are both rounded to
 * bf16 before the next step, as the golden does.
 * ---------------------------------------------------------------------------------------- */
int cmx_mx_gmm_swiglu_quant(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                            const uint8_t* b, const uint8_t* b_scale, uint8_t* act_codes, uint32_t ld_act,
                            uint8_t* act_scales, uint32_t ld_acts, void* act_bf16, const int32_t* group_sizes,
                            uint32_t groups, uint32_t m_total, uint32_t n, uint32_t k, void* workspace,
                            cmx_stream_t stream);

/* cmx_mx_gmm_swiglu_quant without a workspace argument and without any allocation: no counterpart in the
 * reference; it is for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid it).  The tile schedule metadata lives in a fixed array inside the library's device
 * image (33 KiB per device, held until the process ends), which admits at most cmx_mx_gmm_noalloc_max_groups()
 * = 4096 groups; more are rejected with CMX_EINVAL.  All calls on one device share that array: calls that overlap
 * on one device (different streams) race on it; calls on one stream do not.  Same results as
 * cmx_mx_gmm_swiglu_quant.  Under stream capture call cmx_init() beforehand. */
uint32_t cmx_mx_gmm_noalloc_max_groups(void);
int cmx_mx_gmm_swiglu_quant_noalloc(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                    const uint8_t* b, const uint8_t* b_scale, uint8_t* act_codes, uint32_t ld_act,
                                    uint8_t* act_scales, uint32_t ld_acts, void* act_bf16,
                                    const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n,
                                    uint32_t k, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Pre-tiled expert weights (8-bit element formats).  No counterpart in the reference's interface: its operators take
 * the weights in the layout tag the caller names and the AIC block re-tiles them through L1 on every use
 * (include/catccos/dgemm/kernel/ascend950_alltoall_gmm.hpp:193-323).  On this GPU a grouped matmul whose groups hold
 * about one tile of rows streams every weight byte from HBM exactly once, and it does so fastest when each wavefront
 * loads the fragments it multiplies straight into its registers; for that the bytes a wavefront loads together must lie
 * together.  cmx_mx_pretile_weights rewrites dense [groups, n, k] codes ONCE (at weight-load time) into that order:
 *   [group][256-row tile][128-byte K slab][wavefront 0..3][1 KiB load 0..7][lane 0..63][16 bytes]
 * (cmx_mx_pretiled_weight_bytes bytes: groups * tiles * 256 * k, rows past n repeat the last row; 0 for shapes the
 * format does not cover).  pair_gate_up = 1 tiles the weights of cmx_mx_gmm_swiglu_quant, whose tiles pair 128 gate
 * rows with their 128 up rows; 0 those of cmx_mx_gmm.  The scales stay as they are ([groups, n, RoundUp2(k/32)]).
 *
 * cmx_mx_gmm_pretiled / cmx_mx_gmm_swiglu_quant_pretiled are cmx_mx_gmm / cmx_mx_gmm_swiglu_quant with b_tiled in
 * place of b: same arguments otherwise, bit-identical results.  They need what the kernel behind them needs and fail
 * with CMX_EINVAL (nothing launched) otherwise: E4M3 or E5M2, k a multiple of 512, scale rows of both operands
 * 16-byte aligned (pointer and pitch); cmx_mx_gmm_pretiled also a 16-bit output type with n and ldc multiples of 8 and
 * c 16-byte aligned; cmx_mx_gmm_swiglu_quant_pretiled act_bf16 == NULL (codes and scales only).  cmx_dispatch_ffn_combine_pretiled is catccos_ascend950_dispatch_ffn_combine (one device) on
 * w1 tiled with pair_gate_up = 1 and w2 tiled with pair_gate_up = 0; K % 512 == 0 and N % 1024 == 0.
 * Measured at 256 experts x 256 routed rows, K = 7168, N = 4096: GMM1 3 % and GMM2 8 % faster than on row-major
 * weights; with 2048 rows per expert the row-major kernels are the faster ones (the weight stream is shared there).
 * ---------------------------------------------------------------------------------------- */
size_t cmx_mx_pretiled_weight_bytes(uint32_t groups, uint32_t n, uint32_t k, int pair_gate_up);
int cmx_mx_pretile_weights(const uint8_t* b, uint8_t* b_tiled, uint32_t groups, uint32_t n, uint32_t k,
                           int pair_gate_up, cmx_stream_t stream);
int cmx_mx_gmm_pretiled(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b_tiled,
                        const uint8_t* b_scale, void* c, uint32_t ldc, const int32_t* group_sizes, uint32_t groups,
                        uint32_t m_total, uint32_t n, uint32_t k, int fmt, int out_type, void* workspace,
                        cmx_stream_t stream);
int cmx_mx_gmm_swiglu_quant_pretiled(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                     const uint8_t* b_tiled, const uint8_t* b_scale, uint8_t* act_codes,
                                     uint32_t ld_act, uint8_t* act_scales, uint32_t ld_acts, void* act_bf16,
                                     const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n,
                                     uint32_t k, void* workspace, cmx_stream_t stream);
int cmx_dispatch_ffn_combine_pretiled(cmx_stream_t stream, const uint8_t* x, const uint8_t* expertIdx,
                                      const uint8_t* gateWeight, const uint8_t* w1_tiled, const uint8_t* w1Scale,
                                      const uint8_t* w2_tiled, const uint8_t* w2Scale, uint8_t* out, uint8_t* workspace,
                                      uint32_t m, uint32_t k, uint32_t n, uint32_t localExperts, uint32_t topK);

/* ------------------------------------------------------------------------------------------
 * Operands stored with K as the slow axis.
 * The reference's generators write B either transposed ([N, K], what cmx_mx_gemm takes) or as
 * [K, N] codes with scales [K/64, N, 2] (examples/ascend950_mxfp8_matmul_reduce_scatter/scripts/
 * gen_data_mxfp8_mmrs.py:309-330, trans_b = 0: the setting of examples/ascend950_fp8_mx_allgather_matmul,
 * ascend950_mxfp8_matmul_alltoall and ascend950_fp8_mx_alltoallv_grouped_matmul scripts/run.sh:17); A with
 * trans_a = 1 is [K, M] with scales [K/64, M, 2] (:318-321).  On the device these are the RowMajor /
 * ColumnMajor layout tags handed to BlockMmadTla (examples/ascend950_mxfp8_matmul_reduce_scatter/main.cpp:27-32).
 *
 * cmx_mx_to_k_major rewrites `batch` such operands (codes [batch, k, n] with row pitch ld_src, scales
 * [batch, k/64, n, 2] dense) as K-contiguous ones (codes [batch, n, k] with row pitch ld_dst, scales
 * [batch, n, k/32] with row pitch ld_dst_scale).  8-bit element formats; k a multiple of 64.
 * cmx_mxfp4_to_k_major is the same for FP4, where two codes share a byte along the contiguous axis
 * (examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:522-545, 586-620): codes [batch, k, ceil(n/2)] bytes (pairs
 * along n, even column in the low nibble) -> [batch, n, k/2] bytes (pairs along k); pitches in bytes.  The
 * *_ex entry points take CMX_FMT_E2M1 as well (their workspace size functions give the 8-bit size, an upper bound).
 *
 * cmx_mx_gemm_ex / cmx_mx_gmm_ex are cmx_mx_gemm / cmx_mx_gmm for dense operands in either orientation
 * (trans_a = 1: A is [K, M]; trans_b = 0: B is [K, N] resp. [groups, K, N]); operands that are not K-contiguous
 * are normalised into the workspace first (one extra read and write of that operand).  The workspace
 * must be 256-byte aligned and hold *_ex_workspace_bytes bytes (for the grouped form this includes the
 * tile schedule metadata of cmx_mx_gmm).
 * ---------------------------------------------------------------------------------------- */
int cmx_mx_to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst, uint32_t ld_dst,
                      uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n, uint32_t batch,
                      cmx_stream_t stream);
int cmx_mxfp4_to_k_major(const uint8_t* src, uint32_t ld_src, const uint8_t* src_scale, uint8_t* dst, uint32_t ld_dst,
                         uint8_t* dst_scale, uint32_t ld_dst_scale, uint32_t k, uint32_t n, uint32_t batch,
                         cmx_stream_t stream);
size_t cmx_mx_gemm_ex_workspace_bytes(uint32_t m, uint32_t n, uint32_t k, int trans_a, int trans_b);
int cmx_mx_gemm_ex(const uint8_t* a, const uint8_t* a_scale, const uint8_t* b, const uint8_t* b_scale, void* c,
                   uint32_t ldc, uint32_t m, uint32_t n, uint32_t k, int fmt, int out_type, int trans_a, int trans_b,
                   void* workspace, cmx_stream_t stream);
size_t cmx_mx_gmm_ex_workspace_bytes(uint32_t groups, uint32_t n, uint32_t k, int trans_b);
int cmx_mx_gmm_ex(const uint8_t* a, const uint8_t* a_scale, const uint8_t* b, const uint8_t* b_scale, void* c,
                  uint32_t ldc, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n, uint32_t k,
                  int fmt, int out_type, int trans_b, void* workspace, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * INT8 W8A8 grouped matmul with per-channel and per-token dequantisation and SwiGLU: the arithmetic of the
 * reference operator DispatchGmmDequantSwiglu.
 * Replaces AlltoallvGmmDequantKernel + DequantSwigluKernel as composed by AllToAllVGmmDequantSwigluImpl
 * (examples/dispatch_gmm_dequant_swiglu/dispatch_gmm_dequant_swiglu_device.h:60-222) for the rows one
 * device holds; golden examples/utils/gen_data_dispatch_gmm_dequant_swiglu.py:263-320:
 *   c = a_g(int32) @ b_g(int32);  h = fp16(fp32(c) * channel_scale);  y = fp32(h) * token_scale[row];
 *   out = y[:, :n/2] * sigmoid(y[:, :n/2]) * y[:, n/2:]
 *
 *   a              int8 [m_total, k] (expert-sorted rows), pitch lda bytes;  token_scale fp32 [m_total]
 *   b              int8 [groups, k, n] as the reference stores it (trans_b = 0; rewritten K-contiguous in the
 *                  workspace on every call) or [groups, n, k] (trans_b = 1, e.g. rewritten once at load time with
 *                  cmx_bytes_to_k_major)
 *   channel_scale  fp32 [groups * n], one value every channel_scale_stride floats (2 for the reference's file
 *                  of 64-bit words whose low half is the fp32 scale, dispatch_gmm_dequant_swiglu_host.h:26,52-61)
 *   out            [m_total, n/2] of out_type (fp32 as the golden, or fp16 / bf16 as the device writes), pitch
 *                  ld_out elements;  rows past sum(group_sizes) are left untouched
 *   workspace      256-byte aligned, cmx_int8_gmm_workspace_bytes bytes
 * k a multiple of 128, n a multiple of 64.
 *
 * cmx_int8_quant_scatter is the per-token dynamic quantiser in front of it (the quant_mode = 1 leg of the routing
 * routine the golden calls, :159-165; formula :269-274): q = rint(x * 127 / rowmax), scale = rowmax / 127, the row
 * written to each of its top_k destinations src2sorted[t * top_k + r] (negative = skipped; null = identity with
 * top_k = 1).  x bf16 [tokens, k].
 * ---------------------------------------------------------------------------------------- */
int cmx_int8_quant_scatter(const void* x, uint32_t ld_x, const int32_t* src2sorted, int8_t* codes, uint32_t ld_codes,
                           float* scales, uint32_t tokens, uint32_t k, uint32_t top_k, cmx_stream_t stream);
int cmx_bytes_to_k_major(const uint8_t* src, uint32_t ld_src, uint8_t* dst, uint32_t ld_dst, uint32_t k, uint32_t n,
                         uint32_t batch, cmx_stream_t stream);
size_t cmx_int8_gmm_workspace_bytes(uint32_t groups, uint32_t n, uint32_t k, int trans_b);
int cmx_int8_gmm_dequant_swiglu(const int8_t* a, uint32_t lda, const float* token_scale, const int8_t* b,
                                const float* channel_scale, uint32_t channel_scale_stride, void* out, uint32_t ld_out,
                                int out_type, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n,
                                uint32_t k, int trans_b, void* workspace, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * MoE routing: stable sort of (expert, row) pairs.
 * Replaces moe_init_routing_v2 (examples/aux_ops/moe_init_routing_v2/moe_init_routing_v2.h:56-220,
 * moe_v2_src_to_dst_op_simt.h:79-87); golden moe_init_routing_cpu (gen_data_moe.py:48-57).
 *
 *   expert_idx   int32 [tokens, top_k], values in [0, experts)
 *   sorted2src   int32 [tokens*top_k]  = stable argsort of the flattened ids (golden direction)
 *   src2sorted   int32 [tokens*top_k]  = inverse (the device's expandedRowIdx)
 *   counts       int32 [experts]       = rows per expert
 *   workspace    >= cmx_moe_routing_workspace_bytes(tokens*top_k, experts)
 * ---------------------------------------------------------------------------------------- */
size_t cmx_moe_routing_workspace_bytes(uint32_t routes, uint32_t experts);
int cmx_moe_init_routing(const int32_t* expert_idx, uint32_t tokens, uint32_t top_k, uint32_t experts,
                         int32_t* sorted2src, int32_t* src2sorted, int32_t* counts, void* workspace,
                         cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Fused dispatch on one device: quantize each token once (E4M3, RNE) and write the row to its
 * top_k destinations.  Replaces CommBlockMxQuant::QuantScatterPacked
 * (comm_block_mx_quant.hpp:318-368) via QuantScatterRoutingMxFp8
 * (examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h:611-644).
 *
 *   x           bf16 [tokens, k]
 *   src2sorted  int32 [tokens*top_k]; negative destinations are skipped
 *   out_codes   row r at out_codes + r*ld_out; rows 16-byte aligned (ld_out a multiple of 16).
 *   out_scales  row r at out_scales + r*ld_outs.  When the scale rows are 16-byte aligned too they are written in
 *               16-byte pieces: the bytes of a row between its RoundUp2(k/32) columns and the next multiple of 16
 *               are overwritten with zeros, never more -- unless the scale array is an allocation of its own (it
 *               does not overlap [out_codes, out_codes + tokens*top_k*ld_out)) and ld_outs is the next multiple of
 *               128: then the whole pitch is written (data, padding column, zeros), so that no 128-byte line of
 *               the array is written in part.  Callers keep nothing in those bytes.
 * The reference's packed wire row [codes k | scales RoundUp2(k/32) | zero pad to 32 B] is the case
 * out_scales = out_codes + k, ld_out = ld_outs = cmx_packed_row_bytes(k): the zero fill then ends at or before the
 * end of the row's own pad bytes (k is a multiple of 32, so the row has round_up(RoundUp2(k/32), 32) bytes behind
 * its codes), whatever k is.
 * ---------------------------------------------------------------------------------------- */
uint32_t cmx_packed_row_bytes(uint32_t k);
int cmx_quant_scatter(const void* x, uint32_t ld_x, const int32_t* src2sorted, uint8_t* out_codes, uint32_t ld_out,
                      uint8_t* out_scales, uint32_t ld_outs, uint32_t tokens, uint32_t k, uint32_t top_k,
                      cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Weighted top-k combine.  Replaces KernelMoeTokenUnpermute<bf16,int32,float,true>
 * (examples/aux_ops/moe_token_unpermute/moe_token_unpermute.h:233-366):
 * out[t] = bf16( sum_k probs[t,k] * y[src2sorted[t*top_k+k]] ), fp32 multiply then fp32 add in k
 * order; indices outside [0, rows) contribute nothing.
 * ---------------------------------------------------------------------------------------- */
int cmx_moe_token_unpermute(const void* y, uint32_t ld_y, uint32_t rows, const int32_t* src2sorted,
                            const float* probs, void* out, uint32_t ld_out, uint32_t tokens, uint32_t hidden,
                            uint32_t top_k, cmx_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Full single-device MoE FFN: dispatch -> GMM1 -> SwiGLU -> requant -> GMM2 -> combine.
 * Same argument list as CatccosKernel::catccos_ascend950_dispatch_ffn_combine_wrapper
 * (examples/torch_binding/include/catccos_torch_kernel.h:40-44, body
 * examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_wrapper.cpp:18-66) and
 * catccos_ascend950_symmetric_bytes (:24).  blockDim, fftsAddr and symmetric are accepted and
 * ignored (no cube/vector split and no peers on one GPU); rankSize must be 1.
 *
 *   x bf16 [m,k]; expertIdx int32 [m,topK]; gateWeight fp32 [m,topK]
 *   w1 E4M3 [E,n,k], w1Scale [E,n,k/32]; w2 [E,k,n/2], w2Scale [E,k,n/64]; out bf16 [m,k]
 *   workspace >= catccos_ascend950_dispatch_ffn_combine_workspace_bytes(...) ; contents may be
 *   garbage on entry.
 * topK <= min(localExperts, 64), m * topK < 2^31; every shape limit is checked before the first launch.
 * ---------------------------------------------------------------------------------------- */
uint64_t catccos_ascend950_symmetric_bytes(void);
size_t catccos_ascend950_dispatch_ffn_combine_workspace_bytes(uint32_t m, uint32_t k, uint32_t n,
                                                              uint32_t localExperts, uint32_t topK, int rankSize);
int catccos_ascend950_dispatch_ffn_combine(uint32_t blockDim, cmx_stream_t stream, uint64_t fftsAddr,
                                           const uint8_t* x, const uint8_t* expertIdx, const uint8_t* gateWeight,
                                           const uint8_t* w1, const uint8_t* w1Scale, const uint8_t* w2,
                                           const uint8_t* w2Scale, uint8_t* out, uint8_t* workspace,
                                           uint8_t* symmetric, uint32_t m, uint32_t k, uint32_t n,
                                           uint32_t localExperts, uint32_t topK, int rankSize);

/* Offsets of the FFN's intermediate buffers inside the workspace (for tests and debugging). */
typedef struct cmx_ffn_workspace_layout {
    size_t src2sorted, sorted2src, counts, routing_scratch, gmm_meta;
    size_t a_codes, a_scales, act_codes, act_scales, y;
    size_t total;
    size_t a_scales_pitch; /* bytes between the scale rows at a_scales (a multiple of 128, >= RoundUp2(k/32)) */
} cmx_ffn_workspace_layout;
int cmx_ffn_workspace_layout_get(uint32_t m, uint32_t k, uint32_t n, uint32_t localExperts, uint32_t topK,
                                 cmx_ffn_workspace_layout* layout);

#ifdef __cplusplus
}
#endif
#endif /* CATCCOS_MX_H */
