// Block-scaled MX matmul for gfx950 on v_mfma_scale_f32_32x32x64_f8f6f4.
//
//   C[m, n] = sum_k deq(A)[m, k] * deq(W)[n, k]        A = activations, W = transposed weights
//
// Both operands are K-contiguous, which is what the scaled MFMA wants: per step a lane feeds two
// 16-byte runs of one row (FP4: one run = a whole 32-block) plus that row's E8M0 byte for the
// 32-block its half-wave owns.  The weights
// are the MFMA's first operand and the activations the second, so an accumulator register quad
// holds four consecutive n for one m: stores are 8-byte vectors and the SwiGLU/requant epilogue
// finds a whole 32-wide MX block of one activation row in two lanes (l and l^32).
//
// One workgroup (256 threads = 4 wavefronts) owns a TW x TM tile (weight rows x activation rows)
// and walks K in 128-byte slabs through a two-stage LDS ring: while the MFMAs consume slab i
// the global loads of slab i+1 are in flight in registers.  A/W tiles are stored with a 16-byte
// chunk XOR swizzle so both the 16-byte row-strided MFMA operand reads and the staging writes are
// bank-conflict free; the per-row scale dwords of the slab ride along in LDS.
//
// Ragged expert groups: a tiny prologue kernel turns the device-resident group sizes into row
// offsets and a prefix of m-tiles; each workgroup binary-searches its (group, n-tile, m-tile) from
// that prefix, so no host synchronisation is needed and empty groups cost nothing.  Workgroup ids
// are remapped so that each XCD (ids congruent mod 8) walks a contiguous run of tiles that share
// weight panels in its own L2.
#include <atomic>
#include <type_traits>
#include <vector>

#include "mx_common.h"

namespace cmx {

namespace {

constexpr int kSlabBytes = 128;     // K bytes per LDS slab and row
constexpr int kChunks = kSlabBytes / 16;
constexpr int kXcds = 8;

// kEpiStoreBf16 / kEpiStoreFp16: 16-bit output whose rows and row pitch are multiples of eight elements (16-byte
// stores, no per-element edge handling): small enough to sit inside a persistent kernel's tile loop.  Two epilogues, not one with a run-time switch: a second copy of the store loop inside the kernel costs
// registers, and values spilled because of it are reloaded inside the scheduled loop, where the waits that the
// compiler puts behind such reloads drain the operand loads in flight.
// kEpiSwigluQuantAct: kEpiSwigluQuant that also writes the bf16 SwiGLU output (what the tests check the requantised
// codes against).  A kernel of its own for the same reason: the extra output path costs the SwiGLU kernels
// 30 registers, all of them spilled at the tile boundaries, 3 % of a launch, whether the output is asked for or not.
enum Epilogue { kEpiStore = 0, kEpiSwigluQuant = 1, kEpiStoreBf16 = 2, kEpiI8DequantSwiglu = 3, kEpiStoreFp16 = 4, kEpiSwigluQuantAct = 5 };
constexpr bool epi_is_lean_store(int epi) { return epi == kEpiStoreBf16 || epi == kEpiStoreFp16; }
constexpr bool epi_is_swiglu_quant(int epi) { return epi == kEpiSwigluQuant || epi == kEpiSwigluQuantAct; }
// epilogues whose weight tile pairs gate rows (first half of N) with their up partners (second half)
constexpr bool epi_pairs_gate_up(int epi) { return epi_is_swiglu_quant(epi) || epi == kEpiI8DequantSwiglu; }
// element "format" of the INT8 path inside the kernel templates (the public format codes are the MX ones)
constexpr int kFmtI8 = 8;

struct GemmParams {
    const uint8_t* a;        // activations codes
    const uint8_t* a_scale;
    const uint8_t* w;        // weights codes [groups][n][ldw]
    const uint8_t* w_scale;  // [groups][n][ld_ws]
    void* c;
    uint8_t* act_codes;
    uint8_t* act_scales;
    uint16_t* act_bf16;
    const int32_t* row_off;     // [groups+1] (grouped) or null (dense)
    const int32_t* tile_pref;   // [groups+1] prefix of m-tiles (grouped) or null
    int32_t* tile_ctr;          // [8] per-XCD tile counters, zeroed before the launch (persistent grouped 4 x 1 kernels) or null
    uint32_t lda, ld_as, ldw, ld_ws, ldc, ld_act, ld_acts;
    uint32_t m, n, kbytes, kblocks;   // kblocks = K/32
    uint32_t groups, w_tiles;
    int out_type;
    int scale_vec;   // scale rows are 4-byte aligned: one dword load per row and slab
    int scale_vec16; // scale rows are 16-byte aligned: one 16-byte load per row fetches the scales of four slabs
    int w_pretiled;  // w holds the weights in the tiled order of cmx_mx_pretile_weights (the weights-to-registers kernel)
};

__device__ __forceinline__ uint32_t swz(uint32_t row, uint32_t chunk) {
    return chunk ^ ((row & 7u) ^ ((row >> 3) & 1u));
}

__device__ __forceinline__ v4f to_v4(const v16f& v, int q) {
    v4f r = {v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
    return r;
}

template <int FMT>
__device__ __forceinline__ v16f mfma(v8i w, v8i a, v16f c, int opsel_tag, int sw, int sa);

// opsel picks which byte of the lane's scale register feeds the MFMA (same byte for both operands here)
#define CMX_MFMA_CASE(fmtcode, sel) \
    __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, a, c, fmtcode, fmtcode, sel, sw, sel, sa)

template <>
__device__ __forceinline__ v16f mfma<CMX_FMT_E4M3>(v8i w, v8i a, v16f c, int sel, int sw, int sa) {
    switch (sel) {
        case 0: return CMX_MFMA_CASE(0, 0);
        case 1: return CMX_MFMA_CASE(0, 1);
        case 2: return CMX_MFMA_CASE(0, 2);
        default: return CMX_MFMA_CASE(0, 3);
    }
}
template <>
__device__ __forceinline__ v16f mfma<CMX_FMT_E5M2>(v8i w, v8i a, v16f c, int sel, int sw, int sa) {
    switch (sel) {
        case 0: return CMX_MFMA_CASE(1, 0);
        case 1: return CMX_MFMA_CASE(1, 1);
        case 2: return CMX_MFMA_CASE(1, 2);
        default: return CMX_MFMA_CASE(1, 3);
    }
}
template <>
__device__ __forceinline__ v16f mfma<CMX_FMT_E2M1>(v8i w, v8i a, v16f c, int sel, int sw, int sa) {
    switch (sel) {
        case 0: return CMX_MFMA_CASE(4, 0);
        case 1: return CMX_MFMA_CASE(4, 1);
        case 2: return CMX_MFMA_CASE(4, 2);
        default: return CMX_MFMA_CASE(4, 3);
    }
}

// INT8: one 64-deep K step is two v_mfma_i32_32x32x32_i8, fed by the two halves of the same fragment registers
// (any fixed assignment of the 32 K positions to lanes and registers gives the same integer sum, as long as both
// operands use the same one); the INT32 accumulators travel in the fp32 accumulator type bit for bit.
template <>
__device__ __forceinline__ v16f mfma<kFmtI8>(v8i w, v8i a, v16f c, int, int, int) {
    typedef int v16i __attribute__((ext_vector_type(16)));
    v16i acc = __builtin_bit_cast(v16i, c);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8((v4i){w[0], w[1], w[2], w[3]}, (v4i){a[0], a[1], a[2], a[3]}, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8((v4i){w[4], w[5], w[6], w[7]}, (v4i){a[4], a[5], a[6], a[7]}, acc, 0, 0, 0);
    return __builtin_bit_cast(v16f, acc);
}

// g / (1 + exp(-g)) * u with the hardware exponential and reciprocal (about 1 ulp each; the result is rounded
// to bf16 right after)
__device__ __forceinline__ float silu_mul(float g, float u) {
    const float s = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
    return (g * s) * u;
}

struct Tile {
    uint32_t g, mt, wt, row0, rows_valid;
};

// The group tables (row offsets, m-tile prefix) are written by gmm_prepare_kernel before the matmul kernel starts and
// never change under it: reading them through the constant address space lets a wavefront-uniform lookup use scalar
// loads, which wait on lgkmcnt and so do not drain the LDS-DMA loads a persistent kernel has in flight (a vector load
// would: its s_waitcnt vmcnt covers everything issued before it).
__device__ __forceinline__ int32_t table_at(const int32_t* t, uint32_t i) {
    return ((const __attribute__((address_space(4))) int32_t*)t)[i];
}

// Tiles are numbered linearly: within a group m-tiles run fastest so that neighbours share a weight panel;
// dense problems walk bands of four m-tiles across a run of weight tiles.
template <int TM>
__device__ __forceinline__ uint32_t count_m_tiles(const GemmParams& p) {
    return p.row_off != nullptr ? (uint32_t)table_at(p.tile_pref, p.groups) : (p.m + TM - 1) / TM;
}

// Tile L of an XCD-aware order: linear ids congruent mod 8 run on one XCD; each XCD gets a contiguous run.
// Returns the first tile of XCD x and the number of tiles it owns.
__device__ __forceinline__ uint32_t xcd_run(uint32_t total_tiles, uint32_t x, uint32_t& count) {
    const uint32_t base = total_tiles / kXcds, rem = total_tiles % kXcds;
    count = base + (x < rem ? 1u : 0u);
    return x * base + (x < rem ? x : rem);
}

// Persistent kernels that walk in fixed strides (no tile counter), with at least one full round of tiles: instead of
// owning a contiguous run, the XCDs take turns at blocks of (workgroups per XCD) consecutive tiles, workgroup j of XCD x
// walking tiles x * per + j, + grid, + 2 * grid, ...  The whole chip then works on one stretch of `grid` consecutive
// tiles at a time -- two bands of m-tiles across all their weight tiles -- so an activation panel is wanted by four XCDs
// and a weight panel by two at about the same time (the memory-side cache can serve the repeats), and every block of 32
// tiles starts on a multiple of 32, where the contiguous runs cut across the bands.  Zipf-routed 16-expert problem: 16 %
// fewer L2 misses, 1.7-3.3 % less time.  Problems of less than a round keep the contiguous runs, which spread few tiles
// over all eight L2s.
__device__ __forceinline__ void interleave_xcd_walk(uint32_t total_tiles, uint32_t& tile_id, uint32_t& stride, uint32_t& end) {
    if (total_tiles < gridDim.x) return;
    tile_id = (blockIdx.x % kXcds) * (gridDim.x / kXcds) + blockIdx.x / kXcds;
    stride = gridDim.x;
    end = total_tiles;
}

// One tile per workgroup (blockIdx.x < total_tiles).  Workgroups start in the order of their ids, ids congruent mod 8 on one
// XCD.  Whole chunks of 256 tiles: the XCDs take blocks of 32 consecutive tiles of the chunk in turn, for the reason given
// above (the INT8 operator on the 16-expert problem: 973-982 -> 942-945 us); the rest: a contiguous run per XCD.
__device__ __forceinline__ uint32_t tile_of_workgroup(uint32_t total_tiles) {
    constexpr uint32_t kChunk = 32 * kXcds;
    const uint32_t bid = blockIdx.x, full = total_tiles / kChunk * kChunk;
    if (bid < full) return bid / kChunk * kChunk + (bid % kXcds) * 32 + (bid % kChunk) / kXcds;
    uint32_t count;
    const uint32_t k = bid - full;
    return full + xcd_run(total_tiles - full, k % kXcds, count) + k / kXcds;
}

// g_from: a group at or before the tile's (0, or the group of an earlier tile of an increasing sequence)
template <int TM>
__device__ __forceinline__ void decode_tile(const GemmParams& p, uint32_t m_tiles_all, uint32_t L, Tile& t, uint32_t g_from = 0) {
    if (p.row_off != nullptr) {
        // find g with tile_pref[g]*w_tiles <= L < tile_pref[g+1]*w_tiles.  A workgroup's next tile mostly lies in the
        // same group or one of the next two: three independent loads settle that before the bisection's
        // chain of dependent ones
        const uint32_t G = p.groups;
        uint32_t lo = g_from, hi = G;
        const uint32_t i2 = lo + 2 < G ? lo + 2 : G, i3 = lo + 3 < G ? lo + 3 : G;
        const uint32_t t1 = (uint32_t)table_at(p.tile_pref, lo + 1) * p.w_tiles, t2 = (uint32_t)table_at(p.tile_pref, i2) * p.w_tiles,
                       t3 = (uint32_t)table_at(p.tile_pref, i3) * p.w_tiles;
        if (t1 > L) hi = lo + 1;
        else if (t2 > L) { lo += 1; hi = lo + 1; }
        else if (t3 > L) { lo += 2; hi = lo + 1; }
        else lo += 3;
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if ((uint32_t)table_at(p.tile_pref, mid) * p.w_tiles <= L) lo = mid; else hi = mid;
        }
        t.g = lo;
        const uint32_t tp = (uint32_t)table_at(p.tile_pref, lo);
        const uint32_t mtg = (uint32_t)table_at(p.tile_pref, lo + 1) - tp;
        // bands of 8 m-tiles share a run of weight tiles (m fastest inside a band): the 32 tiles that an XCD
        // works on at a time then touch 8 + 4 operand panels instead of mtg + 32/mtg
        const uint32_t local = L - tp * p.w_tiles;
        const uint32_t band = 8;
        const uint32_t per_band = band * p.w_tiles;
        const uint32_t b = local / per_band, within = local % per_band;
        const uint32_t band_rows = (mtg - b * band) < band ? (mtg - b * band) : band;
        t.mt = b * band + within % band_rows;
        t.wt = within / band_rows;
        const uint32_t r_begin = (uint32_t)table_at(p.row_off, lo), r_end = (uint32_t)table_at(p.row_off, lo + 1);
        t.row0 = r_begin + t.mt * TM;
        t.rows_valid = r_end - t.row0 < (uint32_t)TM ? r_end - t.row0 : (uint32_t)TM;
    } else {
        // bands of 4 m-tiles share a run of weight tiles
        const uint32_t band = 4;
        const uint32_t per_band = band * p.w_tiles;
        const uint32_t b = L / per_band, within = L % per_band;
        const uint32_t band_rows = (m_tiles_all - b * band) < band ? (m_tiles_all - b * band) : band;
        t.g = 0;
        t.mt = b * band + within % band_rows;
        t.wt = within / band_rows;
        t.row0 = t.mt * TM;
        t.rows_valid = p.m - t.row0 < (uint32_t)TM ? p.m - t.row0 : (uint32_t)TM;
    }
}

// One tile per workgroup: maps the workgroup id to (group, m-tile, weight tile).  Returns false for ids past
// the last tile.
template <int TM>
__device__ __forceinline__ bool locate_tile(const GemmParams& p, Tile& t) {
    const uint32_t m_tiles_all = count_m_tiles<TM>(p);
    const uint32_t total_tiles = m_tiles_all * p.w_tiles;
    if (blockIdx.x >= total_tiles) return false;
    decode_tile<TM>(p, m_tiles_all, tile_of_workgroup(total_tiles), t);
    return true;
}

// LDS/tile row of a wavefront's weight fragment f (gate fragments first, their up partners second)
template <int TW, int WW, int EPI, int FW>
__device__ __forceinline__ uint32_t wfrag_row_of(uint32_t ww, int f) {
    if (epi_pairs_gate_up(EPI))
        return f < FW / 2 ? ww * (TW / 2 / WW) + f * 32 : TW / 2 + ww * (TW / 2 / WW) + (f - FW / 2) * 32;
    return ww * (TW / WW) + f * 32;
}

template <int TW, int TM, int WW, int WM, int EPI, int FW, int FM>
__device__ __forceinline__ void epilogue(const GemmParams& p, const Tile& tc, v16f (&acc)[FW][FM], uint32_t ww,
                                         uint32_t wm, uint32_t lane) {
    const uint32_t l32 = lane & 31u, lh = lane >> 5;
    const uint32_t wt = tc.wt, row0 = tc.row0, rows_valid = tc.rows_valid;
    auto wfrag_row = [&](int f) -> uint32_t { return wfrag_row_of<TW, WW, EPI, FW>(ww, f); };
    if constexpr (epi_is_lean_store(EPI)) {
        uint16_t* const c = reinterpret_cast<uint16_t*>(p.c);
        auto pack = [](float a, float b) -> uint32_t {
            if constexpr (EPI == kEpiStoreFp16) {
                typedef _Float16 v2h __attribute__((ext_vector_type(2)));
                return __builtin_bit_cast(uint32_t, (v2h){(_Float16)a, (_Float16)b});
            } else {
                return cvt_pk_bf16(a, b);
            }
        };
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
            const uint32_t mloc = wm * (TM / WM) + fm * 32 + l32;
            const bool mvalid = mloc < rows_valid;
            uint16_t* const crow = c + (size_t)(row0 + (mvalid ? mloc : 0)) * p.ldc;
#pragma unroll
            for (int fw = 0; fw < FW; ++fw) {
                // A lane holds columns 8q + 4 lh + {0..3} of its row for q = 0..3, its partner in the other half-wave
                // (same row) the four next to them.  Swapping register halves between the two gives either lane eight
                // consecutive columns: one 16-byte store instead of two 8-byte ones.
#pragma unroll
                for (int qp = 0; qp < 2; ++qp) {
                    const int q = 2 * qp;
                    const uint32_t a0 = pack(acc[fw][fm][4 * q], acc[fw][fm][4 * q + 1]);
                    const uint32_t a1 = pack(acc[fw][fm][4 * q + 2], acc[fw][fm][4 * q + 3]);
                    const uint32_t b0 = pack(acc[fw][fm][4 * q + 4], acc[fw][fm][4 * q + 5]);
                    const uint32_t b1 = pack(acc[fw][fm][4 * q + 6], acc[fw][fm][4 * q + 7]);
                    // upper half of a <-> lower half of b: lower lanes end up with columns 8q .. 8q+7 in (a, b), upper
                    // lanes with 8(q+1) .. 8(q+1)+7
                    const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
                    const uint32_t ncol = wt * TW + wfrag_row(fw) + 8 * (q + lh);
                    if (mvalid && ncol < p.n) *reinterpret_cast<uint4*>(crow + ncol) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                }
            }
        }
    } else if constexpr (EPI == kEpiStore) {
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
            const uint32_t mloc = wm * (TM / WM) + fm * 32 + l32;
            if (mloc >= rows_valid) continue;
            const size_t mrow = (size_t)(row0 + mloc);
#pragma unroll
            for (int fw = 0; fw < FW; ++fw) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t ncol = wt * TW + wfrag_row(fw) + 8 * q + 4 * lh;
                    if (ncol >= p.n) continue;
                    const v4f v = to_v4(acc[fw][fm], q);
                    const bool full = ncol + 4 <= p.n;
                    if (p.out_type == CMX_OUT_BF16) {
                        uint16_t* o = reinterpret_cast<uint16_t*>(p.c) + mrow * p.ldc + ncol;
                        uint32_t b0 = f32_to_bf16(v[0]), b1 = f32_to_bf16(v[1]), b2 = f32_to_bf16(v[2]),
                                 b3 = f32_to_bf16(v[3]);
                        if (full && (p.ldc % 4 == 0)) {
                            *reinterpret_cast<uint2*>(o) = make_uint2(b0 | (b1 << 16), b2 | (b3 << 16));
                        } else {
                            uint32_t bb[4] = {b0, b1, b2, b3};
                            for (uint32_t i = 0; i < 4 && ncol + i < p.n; ++i) o[i] = (uint16_t)bb[i];
                        }
                    } else if (p.out_type == CMX_OUT_FP16) {
                        _Float16* o = reinterpret_cast<_Float16*>(p.c) + mrow * p.ldc + ncol;
                        for (uint32_t i = 0; i < 4 && ncol + i < p.n; ++i) o[i] = (_Float16)v[i];
                    } else {
                        float* o = reinterpret_cast<float*>(p.c) + mrow * p.ldc + ncol;
                        for (uint32_t i = 0; i < 4 && ncol + i < p.n; ++i) o[i] = v[i];
                    }
                }
            }
        }
    } else if constexpr (EPI == kEpiI8DequantSwiglu) {
        // INT32 sums -> fp32 * per-channel scale -> fp16 -> fp32 * per-token scale -> x0 * sigmoid(x0) * gate, fp32 out.
        // w_scale holds the fp32 channel scales of all groups ([groups * n], element stride ld_ws), a_scale the fp32
        // per-row scales.
        typedef int v16i __attribute__((ext_vector_type(16)));
        const uint32_t half = p.n >> 1;
        const float* ch = reinterpret_cast<const float*>(p.w_scale) + (size_t)tc.g * p.n * p.ld_ws;
        const float* ts = reinterpret_cast<const float*>(p.a_scale);
        float* const out = reinterpret_cast<float*>(p.c);
        const bool vec = p.ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(p.c) & 15u) == 0;
#pragma unroll
        for (int f = 0; f < FW / 2; ++f) {
            const uint32_t ncol0 = wt * (TW / 2) + ww * (TW / 2 / WW) + f * 32;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // the four columns 8 q + 4 lh + {0..3} of this fragment: their channel scales serve every row block
                const uint32_t ncol = ncol0 + 8 * q + 4 * lh;
                float cg[4], cu[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t nc = ncol + i < half ? ncol + i : half - 1;
                    cg[i] = ch[(size_t)nc * p.ld_ws];
                    cu[i] = ch[(size_t)(half + nc) * p.ld_ws];
                }
                const bool whole = vec && ncol + 4 <= half;
#pragma unroll
                for (int fm = 0; fm < FM; ++fm) {
                    const uint32_t mloc = wm * (TM / WM) + fm * 32 + l32;
                    if (mloc >= rows_valid) continue;
                    const size_t mrow = (size_t)(row0 + mloc);
                    const float tsv = ts[mrow];
                    const v16i ig = __builtin_bit_cast(v16i, acc[f][fm]), iu = __builtin_bit_cast(v16i, acc[f + FW / 2][fm]);
                    float y[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int r = 4 * q + i;
                        const float x0 = __fmul_rn((float)(_Float16)__fmul_rn((float)ig[r], cg[i]), tsv);
                        const float gate = __fmul_rn((float)(_Float16)__fmul_rn((float)iu[r], cu[i]), tsv);
                        y[i] = __fmul_rn(__fmul_rn(x0, __builtin_amdgcn_rcpf(1.0f + __expf(-x0))), gate);
                    }
                    if (p.out_type == CMX_OUT_FP32) {
                        float* o = out + mrow * p.ldc + ncol;
                        if (whole) {
                            *reinterpret_cast<float4*>(o) = make_float4(y[0], y[1], y[2], y[3]);
                        } else {
                            for (uint32_t i = 0; i < 4 && ncol + i < half; ++i) o[i] = y[i];
                        }
                    } else {
                        uint16_t h[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            h[i] = p.out_type == CMX_OUT_FP16 ? __builtin_bit_cast(uint16_t, (_Float16)y[i]) : (uint16_t)f32_to_bf16(y[i]);
                        uint16_t* o = reinterpret_cast<uint16_t*>(p.c) + mrow * p.ldc + ncol;
                        if (whole) {
                            *reinterpret_cast<uint2*>(o) = make_uint2(h[0] | ((uint32_t)h[1] << 16), h[2] | ((uint32_t)h[3] << 16));
                        } else {
                            for (uint32_t i = 0; i < 4 && ncol + i < half; ++i) o[i] = h[i];
                        }
                    }
                }
            }
        }
    } else {
        const uint32_t half = p.n >> 1;
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
            const uint32_t mloc = wm * (TM / WM) + fm * 32 + l32;
            const bool mvalid = mloc < rows_valid;
            const size_t mrow = (size_t)(row0 + (mvalid ? mloc : 0));
#pragma unroll
            for (int f = 0; f < FW / 2; ++f) {
                // activation column of this fragment's 32-wide MX block
                const uint32_t ncol0 = wt * (TW / 2) + ww * (TW / 2 / WW) + f * 32;
                // GMM1 output rounded to bf16, SwiGLU in fp32, rounded to bf16 again: all on packed pairs with the
                // hardware bf16 conversion; pk[j] holds activation values 2j, 2j+1 of this lane
                uint32_t pk[8];
                uint32_t m = 0;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t g2 = cvt_pk_bf16(acc[f][fm][2 * j], acc[f][fm][2 * j + 1]);
                    const uint32_t u2 = cvt_pk_bf16(acc[f + FW / 2][fm][2 * j], acc[f + FW / 2][fm][2 * j + 1]);
                    const float a0 = silu_mul(__uint_as_float(g2 << 16), __uint_as_float(u2 << 16));
                    const float a1 = silu_mul(__uint_as_float(g2 & 0xFFFF0000u), __uint_as_float(u2 & 0xFFFF0000u));
                    pk[j] = cvt_pk_bf16(a0, a1);
                    m = pk_max_u16(m, pk[j] & 0x7FFF7FFFu);
                }
                if constexpr (EPI == kEpiSwigluQuantAct) {
                    if (p.act_bf16 && mvalid) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const uint32_t ncol = ncol0 + 8 * (r >> 2) + 4 * lh + (r & 3);
                            if (ncol < half) p.act_bf16[mrow * half + ncol] = (uint16_t)(pk[r >> 1] >> (16 * (r & 1)));
                        }
                    }
                }
                uint32_t amax = max(m & 0xFFFFu, m >> 16);
                // the other half of the block's columns sits in lane l ^ 32: swap the half-waves of two copies in the
                // register file (no trip through the LDS crossbar, no lgkmcnt wait between the blocks)
                const auto both = __builtin_amdgcn_permlane32_swap(amax, amax, false, false);
                amax = max(both[0], both[1]);
                const int e = block_exp_from_bf16_amax(amax, kEmaxE4M3);
                if (!mvalid || ncol0 >= half) continue;
                // clamp the magnitudes to 448 * 2^e on the bit patterns, divide by 2^e and cast in one instruction
                const uint32_t lim = (((uint32_t)(e + kEmaxE4M3 + 127) << 7) | 0x60u) * 0x10001u;
                const float scale = __uint_as_float((uint32_t)(e + 127) << 23);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const uint32_t c0 = pk_min_u16(pk[2 * q] & 0x7FFF7FFFu, lim) | (pk[2 * q] & 0x80008000u);
                    const uint32_t c1 = pk_min_u16(pk[2 * q + 1] & 0x7FFF7FFFu, lim) | (pk[2 * q + 1] & 0x80008000u);
                    *reinterpret_cast<uint32_t*>(p.act_codes + mrow * p.ld_act + ncol0 + 8 * q + 4 * lh) =
                        cvt_scaled_pk4<CMX_FMT_E4M3>(c0, c1, scale);
                }
                if (lh == 0) {
                    uint8_t* srow = p.act_scales + mrow * p.ld_acts;
                    const uint32_t blk = ncol0 >> 5;
                    srow[blk] = (uint8_t)(e + 127);
                    const uint32_t nblk = half >> 5;
                    if (blk == nblk - 1 && (nblk & 1u)) srow[nblk] = 127;
                }
            }
        }
    }
}

// The lean 16-bit store in whole cache lines, for the persistent two-slot kernels.  Straight from the accumulator layout
// (epilogue above) a store instruction writes 32 bytes to each of 32 rows and a 128-byte line is complete only after four
// such instructions.  Here the 32 rows x 128 bytes that two neighbouring weight fragments hold for one activation fragment go
// through a 4 KiB staging area in the LDS (16-byte pieces, XOR-swizzled by row: neither the writes nor the reads conflict)
// and come back with eight lanes on a row, so that a store instruction writes eight whole lines, non-temporal (the kernel
// does not read its output again).  `stage` is the wavefront's own 4 KiB; a wavefront reads only what it wrote itself.
template <int TW, int TM, int WW, int WM, int EPI, int FW, int FM>
__device__ __forceinline__ void lean_store_lines(const GemmParams& p, const Tile& tc, v16f (&acc)[FW][FM], uint32_t ww, uint32_t wm,
                                                 uint32_t lane, uint32_t stage) {
    static_assert(epi_is_lean_store(EPI) && FW % 2 == 0, "16-bit store epilogues, weight fragments in pairs");
    const uint32_t l32 = lane & 31u, lh = lane >> 5;
    auto pack = [](float a, float b) -> uint32_t {
        if constexpr (EPI == kEpiStoreFp16) {
            typedef _Float16 v2h __attribute__((ext_vector_type(2)));
            return __builtin_bit_cast(uint32_t, (v2h){(_Float16)a, (_Float16)b});
        } else {
            return cvt_pk_bf16(a, b);
        }
    };
    // write side: row l32 of the fragment, piece (f2, qp, lh) = columns 32 f2 + 16 qp + 8 lh .. + 8 of the pair's 64
    const uint32_t wr_row = stage + l32 * 128;
    // read side: instruction j covers rows 8 j .. 8 j + 7, lane i row 8 j + i / 8, piece i % 8
    const uint32_t rd_r = lane >> 3, rd_p = lane & 7u;
    uint16_t* const c = reinterpret_cast<uint16_t*>(p.c);
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
#pragma unroll
        for (int pr = 0; pr < FW / 2; ++pr) {
#pragma unroll
            for (int f2 = 0; f2 < 2; ++f2) {
                const int fw = 2 * pr + f2;
#pragma unroll
                for (int qp = 0; qp < 2; ++qp) {
                    const int q = 2 * qp;
                    const uint32_t a0 = pack(acc[fw][fm][4 * q], acc[fw][fm][4 * q + 1]);
                    const uint32_t a1 = pack(acc[fw][fm][4 * q + 2], acc[fw][fm][4 * q + 3]);
                    const uint32_t b0 = pack(acc[fw][fm][4 * q + 4], acc[fw][fm][4 * q + 5]);
                    const uint32_t b1 = pack(acc[fw][fm][4 * q + 6], acc[fw][fm][4 * q + 7]);
                    // upper half of a <-> lower half of b: either lane ends up with eight consecutive columns of its row
                    const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
                    const uint32_t piece = 4 * f2 + 2 * qp + lh;
                    const uint32_t addr = wr_row + ((piece ^ (l32 & 7u)) << 4);
                    asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"((v4i){(int)s0[0], (int)s1[0], (int)s0[1], (int)s1[1]}) : "memory");
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            v4i v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t r = 8 * j + rd_r;
                asm volatile("ds_read_b128 %0, %1" : "=v"(v[j]) : "v"(stage + r * 128 + ((rd_p ^ (r & 7u)) << 4)) : "memory");
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // also: the area is free for the next pair's pieces
            const uint32_t col = tc.wt * TW + ww * (TW / WW) + pr * 64 + rd_p * 8;      // first of the lane's eight output columns
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t mloc = wm * (TM / WM) + fm * 32 + 8 * j + rd_r;
                if (mloc < tc.rows_valid && col < p.n)                   // n is a multiple of 8: a piece is in or out as a whole
                    __builtin_nontemporal_store(v[j], reinterpret_cast<v4i*>(c + (size_t)(tc.row0 + mloc) * p.ldc + col));
            }
        }
    }
}

// TW/TM: tile rows (weights / activations); WW x WM wavefront grid over the tile (4 or 8 wavefronts).
// FAST: K is a whole number of slabs and scale rows are dword aligned, so the main loop carries no
// bounds checks at all.
template <int FMT, int TW, int TM, int WW, int WM, int EPI, bool FAST>
__global__ __launch_bounds__(64 * WW * WM) void mx_gemm_kernel(const GemmParams p) {
    constexpr int NT = 64 * WW * WM;
    static_assert(NT == 256 || NT == 512, "four or eight wavefronts per workgroup");
    constexpr bool kFp4 = FMT == CMX_FMT_E2M1;
    constexpr int kSub = kFp4 ? 4 : 2;                 // MFMA steps (64 K elements each) per slab
    constexpr int kScaleDw = kFp4 ? 2 : 1;             // scale dwords per row per slab
    constexpr int FW = TW / WW / 32;                   // 32-row fragments per wavefront, weights
    constexpr int FM = TM / WM / 32;                   // activations
    constexpr int kRowsPerPass = NT / kChunks;         // tile rows covered by one 16-byte load per thread
    constexpr int kWLoads = TW / kRowsPerPass;         // 16-byte chunks per thread per slab
    constexpr int kALoads = TM / kRowsPerPass;
    static_assert(FW >= 1 && FM >= 1 && kWLoads >= 1 && kALoads >= 1, "tile too small for the wavefront grid");
    static_assert(!epi_pairs_gate_up(EPI) || (FW % 2 == 0), "gate/up fragments come in pairs");
    static_assert(TW <= NT && TM <= NT, "one scale row per thread");
    constexpr int kStageBytes = (TW + TM) * kSlabBytes + (TW + TM) * 4 * kScaleDw;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const uint32_t ww = wave % WW, wm = wave / WW;

    Tile tc;
    if (!locate_tile<TM>(p, tc)) return;
    const uint32_t g = tc.g, wt = tc.wt, row0 = tc.row0, rows_valid = tc.rows_valid;

    // ---- global -> LDS staging assignments -----------------------------------------------------
    const uint32_t ld_chunk = tid & 7u;                // 16-byte chunk inside the slab
    const uint32_t ld_row = tid >> 3;                  // + kRowsPerPass*j
    const uint8_t* wg = p.w + (size_t)g * p.n * p.ldw;             // uniform bases, 32-bit lane offsets
    const uint8_t* wsg = p.w_scale + (size_t)g * p.n * p.ld_ws;
    const uint8_t* ag = p.a + (size_t)row0 * p.lda;
    const uint8_t* asg = p.a_scale + (size_t)row0 * p.ld_as;

    // global weight row of LDS tile row r (rows past the matrix repeat the last one; masked at the store)
    auto wrow_of = [&](uint32_t r) -> uint32_t {
        uint32_t gr;
        if (epi_pairs_gate_up(EPI)) {
            const uint32_t half = p.n >> 1;
            uint32_t rr = r < TW / 2 ? wt * (TW / 2) + r : wt * (TW / 2) + (r - TW / 2);
            rr = rr < half ? rr : half - 1;
            gr = r < TW / 2 ? rr : half + rr;
        } else {
            gr = wt * TW + r;
            gr = gr < p.n ? gr : p.n - 1;
        }
        return gr;
    };
    auto arow_of = [&](uint32_t r) -> uint32_t { return r < rows_valid ? r : rows_valid - 1; };

    uint32_t woff[kWLoads], aoff[kALoads];
#pragma unroll
    for (int j = 0; j < kWLoads; ++j) woff[j] = wrow_of(ld_row + kRowsPerPass * j) * p.ldw + ld_chunk * 16;
#pragma unroll
    for (int j = 0; j < kALoads; ++j) aoff[j] = arow_of(ld_row + kRowsPerPass * j) * p.lda + ld_chunk * 16;
    // scale rows: thread t serves weight row t (t < TW) and activation row t (t < TM)
    const uint32_t wsoff = wrow_of(tid < TW ? tid : 0) * p.ld_ws;
    const uint32_t asoff = arow_of(tid < TM ? tid : 0) * p.ld_as;

    const uint32_t nslab = (p.kbytes + kSlabBytes - 1) / kSlabBytes;
    constexpr uint32_t blocks_per_slab = 4 * kScaleDw;

    uint4 wreg[kWLoads], areg[kALoads];
    uint32_t wsreg[kScaleDw], asreg[kScaleDw];

    auto load_scale_dw = [&](const uint8_t* rowp, uint32_t blk0) -> uint32_t {
        // four consecutive scale bytes starting at block blk0; beyond K the scale is 1.0
        if (FAST || (p.scale_vec && blk0 + 4 <= p.kblocks)) return *reinterpret_cast<const uint32_t*>(rowp + blk0);
        uint32_t v = 0x7F7F7F7Fu;
        for (uint32_t i = 0; i < 4; ++i)
            if (blk0 + i < p.kblocks) v = (v & ~(0xFFu << (8 * i))) | ((uint32_t)rowp[blk0 + i] << (8 * i));
        return v;
    };
    auto load_global = [&](uint32_t slab) {
        const uint8_t* wslab = wg + (size_t)slab * kSlabBytes;
        const uint8_t* aslab = ag + (size_t)slab * kSlabBytes;
        const bool in = FAST || (slab * kSlabBytes + ld_chunk * 16 < p.kbytes);
#pragma unroll
        for (int j = 0; j < kWLoads; ++j)
            wreg[j] = in ? *reinterpret_cast<const uint4*>(wslab + woff[j]) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < kALoads; ++j)
            areg[j] = in ? *reinterpret_cast<const uint4*>(aslab + aoff[j]) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int d = 0; d < kScaleDw; ++d) {
            const uint32_t blk0 = slab * blocks_per_slab + 4 * d;
            if (tid < TW) wsreg[d] = load_scale_dw(wsg + wsoff, blk0);
            if (tid < TM) asreg[d] = load_scale_dw(asg + asoff, blk0);
        }
    };
    auto store_lds = [&](uint32_t stage) {
        uint8_t* sW = smem + stage * kStageBytes;
        uint8_t* sA = sW + TW * kSlabBytes;
        uint32_t* sWs = reinterpret_cast<uint32_t*>(sA + TM * kSlabBytes);
        uint32_t* sAs = sWs + TW * kScaleDw;
#pragma unroll
        for (int j = 0; j < kWLoads; ++j) {
            const uint32_t r = ld_row + kRowsPerPass * j;
            *reinterpret_cast<uint4*>(sW + r * kSlabBytes + swz(r, ld_chunk) * 16) = wreg[j];
        }
#pragma unroll
        for (int j = 0; j < kALoads; ++j) {
            const uint32_t r = ld_row + kRowsPerPass * j;
            *reinterpret_cast<uint4*>(sA + r * kSlabBytes + swz(r, ld_chunk) * 16) = areg[j];
        }
#pragma unroll
        for (int d = 0; d < kScaleDw; ++d) {
            if (tid < TW) sWs[tid * kScaleDw + d] = wsreg[d];
            if (tid < TM) sAs[tid * kScaleDw + d] = asreg[d];
        }
    };

    // ---- accumulators --------------------------------------------------------------------------
    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    auto wfrag_row = [&](int f) -> uint32_t { return wfrag_row_of<TW, WW, EPI, FW>(ww, f); };
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    // byte offsets (within a stage's W / A tile) of the lane's two 16-byte runs for step 0; the runs
    // of step h sit at chunk index + 4h (8-bit) or + 2h (FP4), i.e. the XOR swizzle is re-applied
    auto frag_addr = [&](uint32_t r, uint32_t c) -> uint32_t { return r * kSlabBytes + swz(r, c) * 16; };

    auto read_frag = [&](const uint8_t* tile, uint32_t r, int h) -> v8i {
        if (kFp4) {
            v4i lo = *reinterpret_cast<const v4i*>(tile + frag_addr(r, h * 2 + lh));
            return (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
        }
        // 8-bit operands: registers 0-3 carry k = 16*lh + [0,16) of the step's first 32-block,
        // registers 4-7 the same slice of its second 32-block
        v4i lo = *reinterpret_cast<const v4i*>(tile + frag_addr(r, h * 4 + lh));
        v4i hi = *reinterpret_cast<const v4i*>(tile + frag_addr(r, h * 4 + lh + 2));
        return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    auto compute = [&](uint32_t stage) {
        const uint8_t* sW = smem + stage * kStageBytes;
        const uint8_t* sA = sW + TW * kSlabBytes;
        const uint32_t* sWs = reinterpret_cast<const uint32_t*>(sA + TM * kSlabBytes);
        const uint32_t* sAs = sWs + TW * kScaleDw;
        // operand fragments are double buffered in registers: the LDS reads of step h+1 are issued
        // before the MFMAs of step h
        v8i af[2][FM], wf[2][FW];
#pragma unroll
        for (int f = 0; f < FM; ++f) af[0][f] = read_frag(sA, wm * (TM / WM) + f * 32 + l32, 0);
#pragma unroll
        for (int f = 0; f < FW; ++f) wf[0][f] = read_frag(sW, wfrag_row(f) + l32, 0);
        // lane's scale registers: byte 2*h' (after the lh shift) belongs to MFMA step h' of the dword
        uint32_t sw[FW][kScaleDw], sa[FM][kScaleDw];
#pragma unroll
        for (int f = 0; f < FW; ++f)
#pragma unroll
            for (int d = 0; d < kScaleDw; ++d) sw[f][d] = sWs[(wfrag_row(f) + l32) * kScaleDw + d] >> (8 * lh);
#pragma unroll
        for (int f = 0; f < FM; ++f)
#pragma unroll
            for (int d = 0; d < kScaleDw; ++d)
                sa[f][d] = sAs[(wm * (TM / WM) + f * 32 + l32) * kScaleDw + d] >> (8 * lh);

#pragma unroll
        for (int h = 0; h < kSub; ++h) {
            const int cur = h & 1, nxt = cur ^ 1;
            if (h + 1 < kSub) {
#pragma unroll
                for (int f = 0; f < FM; ++f) af[nxt][f] = read_frag(sA, wm * (TM / WM) + f * 32 + l32, h + 1);
#pragma unroll
                for (int f = 0; f < FW; ++f) wf[nxt][f] = read_frag(sW, wfrag_row(f) + l32, h + 1);
            }
#pragma unroll
            for (int fw = 0; fw < FW; ++fw) {
#pragma unroll
                for (int fm = 0; fm < FM; ++fm) {
                    // step h uses scale dword h/2, byte 2*(h%2) of the shifted register
                    acc[fw][fm] = mfma<FMT>(wf[cur][fw], af[cur][fm], acc[fw][fm], (h & 1) * 2, (int)sw[fw][h >> 1],
                                            (int)sa[fm][h >> 1]);
                }
            }
        }
    };

    // ---- main loop -------------------------------------------------------------------------------
    load_global(0);
    store_lds(0);
    __syncthreads();
    // steady state is branch free: prefetch slab s+1, consume slab s, refill the other stage
    for (uint32_t s = 0; s + 1 < nslab; ++s) {
        load_global(s + 1);
        __builtin_amdgcn_sched_barrier(0);
        compute(s & 1u);
        // Keep the LDS refill (which waits for the global loads) behind the MFMAs of this slab: without
        // a use of the accumulators here the compiler sinks the MFMAs below the refill and the barrier,
        // which exposes the whole global-load latency every iteration.
#pragma unroll
        for (int i = 0; i < FW; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j) asm volatile("" ::"a"(acc[i][j][0]) : "memory");
        __builtin_amdgcn_sched_barrier(0);
        store_lds((s + 1) & 1u);
        __syncthreads();
    }
    compute((nslab - 1) & 1u);

    epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
}

// ------------------------------------------------------------------------------------------------
// Streaming kernel: operand tiles go global -> LDS directly (LDS-DMA loads, no staging registers and
// no ds_write) into a two-slot ring of 128-byte-deep K slabs; whole 128-byte lines per row keep every
// fetched cache line fully used.  Operand fragments are prefetched into a spare register set one MFMA
// step ahead, so a slot is drained one step before its slab's MFMAs end; at that point
//   wait (own reads of slot s and own loads of slab s+1 done) -> barrier (everyone's) ->
//   refill slot s with slab s+2 -> read the first fragments of slab s+1 -> last MFMA step of slab s.
// One barrier per slab; every load has a full slab of MFMA time to land.
// A load instruction of one wavefront fills 1 KiB of LDS linearly (lane p -> 16 bytes at 16p), i.e.
// 8 tile rows x 8 chunks; the XOR swizzle that keeps the row-strided fragment reads conflict-free is
// applied on the global side (which 16 bytes of the row a lane fetches).  Scale dwords (4 blocks each)
// ride in their own two-slot ring.
#define CMX_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)
#define CMX_WAIT_ALL() __builtin_amdgcn_s_waitcnt(0x0070)   // vmcnt(0) lgkmcnt(0)

typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(1))) void* global_void_ptr;

template <int FMT, int TW, int TM, int WW, int WM, int EPI>
__global__ __launch_bounds__(64 * WW * WM) void mx_gemm_dl_kernel(const GemmParams p) {
    constexpr int NW = WW * WM;                        // wavefronts: 4 (one per SIMD) or 8 (two per SIMD)
    static_assert(NW == 4 || NW == 8, "four or eight wavefronts per workgroup");
    constexpr bool kFp4 = FMT == CMX_FMT_E2M1;
    constexpr bool kI8 = FMT == kFmtI8;                // INT8: no block scales at all
    constexpr int kSub = kFp4 ? 4 : 2;                 // MFMA steps (64 K elements each) per slab
    constexpr int kScaleDw = kI8 ? 0 : (kFp4 ? 2 : 1); // scale dwords per row per slab
    constexpr int kScaleDwA = kScaleDw ? kScaleDw : 1; // array extent
    constexpr int FW = TW / WW / 32, FM = TM / WM / 32;
    constexpr int kRows = TW + TM;                     // W tile rows then A tile rows
    constexpr int kTileLoads = kRows / (8 * NW);       // direct loads per thread and slab (8 rows per wavefront-load)
    constexpr int kWTileLoads = TW / (8 * NW);
    constexpr int kSlotBytes = kRows * kSlabBytes;
    constexpr int kScaleSlot = kRows * kScaleDw;       // dwords
    constexpr int kScaleWaveLoads = kRows / 64;        // wavefront-loads that cover one scale dword of every row
    constexpr int kScalePerWave = (kScaleWaveLoads + NW - 1) / NW;
    constexpr int kLoadsPerSlab = kTileLoads + kScalePerWave * kScaleDw;
    static_assert(TW % (8 * NW) == 0 && TM % (8 * NW) == 0 && TW % 64 == 0 && TM % 64 == 0, "tile shape");
    static_assert(FW >= 1 && FM >= 1, "tile too small for the wavefront grid");
    static_assert(!epi_pairs_gate_up(EPI) || (FW % 2 == 0), "gate/up fragments come in pairs");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint32_t* const sScale = reinterpret_cast<uint32_t*>(smem + 2 * kSlotBytes);

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t ww = wave % WW, wm = wave / WW;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    Tile tc;
    if (!locate_tile<TM>(p, tc)) return;
    const uint32_t g = __builtin_amdgcn_readfirstlane(tc.g), wt = __builtin_amdgcn_readfirstlane(tc.wt);
    const uint32_t row0 = __builtin_amdgcn_readfirstlane(tc.row0);
    const uint32_t rows_valid = __builtin_amdgcn_readfirstlane(tc.rows_valid);

    const uint8_t* wg = p.w + (size_t)g * p.n * p.ldw;
    const uint8_t* wsg = p.w_scale + (size_t)g * p.n * p.ld_ws;
    const uint8_t* ag = p.a + (size_t)row0 * p.lda;
    const uint8_t* asg = p.a_scale + (size_t)row0 * p.ld_as;

    auto wrow_of = [&](uint32_t r) -> uint32_t {
        uint32_t gr;
        if (epi_pairs_gate_up(EPI)) {
            const uint32_t half = p.n >> 1;
            uint32_t rr = r < TW / 2 ? wt * (TW / 2) + r : wt * (TW / 2) + (r - TW / 2);
            rr = rr < half ? rr : half - 1;
            gr = r < TW / 2 ? rr : half + rr;
        } else {
            gr = wt * TW + r;
            gr = gr < p.n ? gr : p.n - 1;
        }
        return gr;
    };
    auto arow_of = [&](uint32_t r) -> uint32_t { return r < rows_valid ? r : rows_valid - 1; };

    // ---- per-lane offsets of the direct loads --------------------------------------------------
    // load i of this wavefront fills combined tile rows (NW*i + wave)*8 .. +8; lane p -> row +p/8, LDS chunk p%8
    uint32_t goff[kTileLoads];
#pragma unroll
    for (int i = 0; i < kTileLoads; ++i) {
        const uint32_t cr = (NW * i + wave) * 8 + (lane >> 3);
        const uint32_t logical = swz(cr, lane & 7u);
        goff[i] = (i < kWTileLoads ? wrow_of(cr) * p.ldw : arow_of(cr - TW) * p.lda) + logical * 16;
    }
    // scale dwords: one wavefront-load covers 64 rows; wavefront-load j serves W rows 64j.. (j < TW/64) or A rows
    uint32_t soff_[kScalePerWave], sdst_[kScalePerWave];
    bool s_is_w[kScalePerWave];
#pragma unroll
    for (int t = 0; t < kScalePerWave; ++t) {
        const uint32_t j = wave + NW * t;
        s_is_w[t] = j < TW / 64;
        const uint32_t aj = (j - TW / 64) % (TM / 64);
        soff_[t] = s_is_w[t] ? wrow_of(64 * j + lane) * p.ld_ws : arow_of(64 * aj + lane) * p.ld_as;
        sdst_[t] = s_is_w[t] ? 64 * j : TW + 64 * aj;
    }

    const uint32_t nslab = p.kbytes / kSlabBytes;

    // Buffer addressing: per-lane byte offsets stay constant over the whole K loop and the slab
    // position is a scalar offset, so a load costs no vector ALU work at all.
    constexpr int kRsrcFlags = 0x00020000;
    auto uniform_ptr = [](const uint8_t* q) -> uint8_t* {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
        return reinterpret_cast<uint8_t*>(((uint64_t)hi << 32) | lo);
    };
    const __amdgpu_buffer_rsrc_t w_rs = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(wg), 0, -1, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(ag), 0, -1, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t ws_rs = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(wsg), 0, -1, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t as_rs = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(asg), 0, -1, kRsrcFlags);

    auto issue_slab = [&](uint32_t slab) {
        const uint32_t k = slab < nslab ? slab : nslab - 1;              // past the end: harmless reload
        uint8_t* dst = smem + (slab & 1u) * kSlotBytes + wave * 1024;
        const int koff = (int)(k * kSlabBytes);
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(i < kWTileLoads ? w_rs : a_rs, (lds_void_ptr)(dst + i * (NW * 1024)), 16,
                                                     (int)goff[i], koff, 0, 0);
        }
        uint32_t* sdst = sScale + (slab & 1u) * kScaleSlot;
#pragma unroll
        for (int d = 0; d < kScaleDw; ++d) {
            const int soff = (int)((k * kScaleDw + d) * 4);
#pragma unroll
            for (int t = 0; t < kScalePerWave; ++t) {
                if (s_is_w[t])
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(ws_rs, (lds_void_ptr)(sdst + d * kRows + sdst_[t]), 4, (int)soff_[t], soff, 0, 0);
                else
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(as_rs, (lds_void_ptr)(sdst + d * kRows + sdst_[t]), 4, (int)soff_[t], soff, 0, 0);
            }
        }
    };

    // ---- fragment reads ------------------------------------------------------------------------
    auto wfrag_row = [&](int f) -> uint32_t { return wfrag_row_of<TW, WW, EPI, FW>(ww, f); };
    auto read_frag = [&](const uint8_t* tile, uint32_t r, int h) -> v8i {
        const uint8_t* rp = tile + r * kSlabBytes;
        if (kFp4) {
            v4i lo = *reinterpret_cast<const v4i*>(rp + swz(r, h * 2 + lh) * 16);
            return (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
        }
        // 8-bit operands: registers 0-3 carry k = 16*lh + [0,16) of the step's first 32-block,
        // registers 4-7 the same slice of its second 32-block
        v4i lo = *reinterpret_cast<const v4i*>(rp + swz(r, h * 4 + lh) * 16);
        v4i hi = *reinterpret_cast<const v4i*>(rp + swz(r, h * 4 + lh + 2) * 16);
        return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    v8i wf[2][FW], af[2][FM];
    uint32_t sw[kScaleDwA][FW] = {}, sa[kScaleDwA][FM] = {}, swn[kScaleDwA][FW] = {}, san[kScaleDwA][FM] = {};

    auto read_frags = [&](uint32_t slab, int h, int buf) {
        const uint8_t* st = smem + (slab & 1u) * kSlotBytes;
#pragma unroll
        for (int f = 0; f < FM; ++f) af[buf][f] = read_frag(st + TW * kSlabBytes, wm * (TM / WM) + f * 32 + l32, h);
#pragma unroll
        for (int f = 0; f < FW; ++f) wf[buf][f] = read_frag(st, wfrag_row(f) + l32, h);
    };
    auto read_scales = [&](uint32_t slab, uint32_t (&w_)[kScaleDwA][FW], uint32_t (&a_)[kScaleDwA][FM]) {
        const uint32_t* sc = sScale + (slab & 1u) * kScaleSlot;
#pragma unroll
        for (int d = 0; d < kScaleDw; ++d) {
#pragma unroll
            for (int f = 0; f < FW; ++f) w_[d][f] = sc[d * kRows + wfrag_row(f) + l32] >> (8 * lh);
#pragma unroll
            for (int f = 0; f < FM; ++f) a_[d][f] = sc[d * kRows + TW + wm * (TM / WM) + f * 32 + l32] >> (8 * lh);
        }
    };

    // ---- prologue -----------------------------------------------------------------------------------
    issue_slab(0);
    issue_slab(1);
    CMX_WAIT_VMCNT(kLoadsPerSlab);      // slab 0 has landed (slab 1 may still be in flight)
    __syncthreads();
    read_frags(0, 0, 0);
    read_scales(0, sw, sa);

    for (uint32_t s = 0; s < nslab; ++s) {
#pragma unroll
        for (int h = 0; h < kSub; ++h) {
            if (h + 1 < kSub) {
                read_frags(s, h + 1, (h + 1) & 1);
            } else {
                // slot s&1 is drained by this wavefront one step early: refill point
                CMX_WAIT_ALL();                 // own fragment reads of slab s and own loads of slab s+1 are done
                __syncthreads();                // ... and everyone else's
                issue_slab(s + 2);
                read_frags(s + 1, 0, 0);
                read_scales(s + 1, swn, san);
            }
            // One wavefront per SIMD issues in order, so the MFMA pipe idles whenever more than one
            // MFMA time of other instructions sits between two MFMAs: spread the LDS reads and the
            // LDS-DMA loads of this step evenly behind the MFMAs instead of clustering them.
            {
                constexpr int kMfmas = FW * FM * (kI8 ? 2 : 1);
                constexpr int kFragReads = (FW + FM) * (kFp4 ? 1 : 2);
                constexpr int kDs = kFragReads + (FW + FM) * kScaleDw;     // refill step also reads the scales
                constexpr int kDsPer = (kDs + kMfmas - 1) / kMfmas;
                constexpr int kVmPer = (kLoadsPerSlab + kMfmas - 1) / kMfmas;
#pragma unroll
                for (int i = 0; i < kMfmas; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);          // one MFMA
                    if (h + 1 == kSub) __builtin_amdgcn_sched_group_barrier(0x020, kVmPer, 0);   // VMEM reads
                    __builtin_amdgcn_sched_group_barrier(0x100, kDsPer, 0);     // DS reads
                }
            }
#pragma unroll
            for (int fw = 0; fw < FW; ++fw)
#pragma unroll
                for (int fm = 0; fm < FM; ++fm)
                    acc[fw][fm] = mfma<FMT>(wf[h & 1][fw], af[h & 1][fm], acc[fw][fm], (h & 1) * 2, (int)sw[h >> 1][fw],
                                            (int)sa[h >> 1][fm]);
            // ... and this step's MFMAs must be issued before the next step's wait/barrier
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int d = 0; d < kScaleDw; ++d) {
#pragma unroll
            for (int f = 0; f < FW; ++f) sw[d][f] = swn[d][f];
#pragma unroll
            for (int f = 0; f < FM; ++f) sa[d][f] = san[d][f];
        }
    }
    CMX_WAIT_VMCNT(0);      // the two reloads issued past the end must land before the LDS is released

    epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
}

#include "mx_gemm_pipe.h"
#include "mx_gemm_wreg.h"
#include "mx_gemm_pipe_fp4.h"

// Row offsets and m-tile prefix of the groups (one workgroup of 256 threads): each thread owns a contiguous run of
// groups; the 256 partial sums are scanned in LDS, first for the rows, then for the m-tiles.
// Group sizes live on the device, so the host cannot check them: negative sizes count as zero and rows past
// m_total (the rows the caller's buffers hold) are cut off here, so that no tile ever points outside them.
__global__ __launch_bounds__(256) void gmm_prepare_kernel(const int32_t* __restrict__ sizes, uint32_t groups, uint32_t tile_m,
                                                           uint32_t m_total, int32_t* __restrict__ row_off,
                                                           int32_t* __restrict__ tile_pref, int32_t* __restrict__ tile_ctr) {
    __shared__ unsigned long long part_r[256];
    __shared__ int32_t part_t[256];
    if (threadIdx.x < kXcds) tile_ctr[threadIdx.x] = 0;
    const uint32_t per = (groups + 255) / 256;
    const uint32_t lo = threadIdx.x * per < groups ? threadIdx.x * per : groups;
    const uint32_t hi = lo + per < groups ? lo + per : groups;
    auto size_of = [&](uint32_t i) -> unsigned long long {
        const int32_t c = sizes[i];
        return c > 0 ? (unsigned long long)c : 0ull;
    };
    // inclusive scan of part[0..255] in place: within each wavefront by lane shuffles, then the three wavefront totals
    // before it added to every element (two barriers instead of sixteen)
    auto scan256 = [&](auto* part) {
        auto v = part[threadIdx.x];
        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const auto u = __shfl_up(v, d);
            if (lane >= (uint32_t)d) v += u;
        }
        part[threadIdx.x] = v;
        __syncthreads();
        decltype(v) before = 0;
        for (uint32_t w = 0; w < wave; ++w) before += part[64 * w + 63];
        __syncthreads();
        part[threadIdx.x] = v + before;
        __syncthreads();
    };
    unsigned long long r = 0;
    for (uint32_t i = lo; i < hi; ++i) r += size_of(i);
    part_r[threadIdx.x] = r;
    __syncthreads();
    scan256(part_r);
    const unsigned long long r_base = threadIdx.x ? part_r[threadIdx.x - 1] : 0ull;
    // rows of group i that fit below m_total, given the rows before it
    auto clipped = [&](unsigned long long before, unsigned long long c) -> uint32_t {
        const unsigned long long b = before < m_total ? before : m_total;
        const unsigned long long e = before + c < m_total ? before + c : m_total;
        return (uint32_t)(e - b);
    };
    r = r_base;
    int32_t t = 0;
    for (uint32_t i = lo; i < hi; ++i) {
        const unsigned long long c = size_of(i);
        t += (int32_t)((clipped(r, c) + tile_m - 1) / tile_m);
        r += c;
    }
    part_t[threadIdx.x] = t;
    __syncthreads();
    scan256(part_t);
    r = r_base;
    t = threadIdx.x ? part_t[threadIdx.x - 1] : 0;
    for (uint32_t i = lo; i < hi; ++i) {
        const unsigned long long c = size_of(i);
        row_off[i] = (int32_t)(r < m_total ? r : m_total);
        tile_pref[i] = t;
        t += (int32_t)((clipped(r, c) + tile_m - 1) / tile_m);
        r += c;
    }
    if (threadIdx.x == 255) {
        const unsigned long long all = part_r[255];
        row_off[groups] = (int32_t)(all < m_total ? all : m_total);
        tile_pref[groups] = part_t[255];
    }
}

// Launch state that belongs to a device, not to the process: the dynamic-LDS limit of a kernel has to be raised on
// every device that runs it, and the CU count differs between devices.  One slot per device ordinal; the flags are
// atomics so that concurrent first calls from several host threads are merely redundant.
constexpr int kMaxDevices = 64;

struct PerDeviceFlag {
    std::atomic<bool> done[kMaxDevices];
};

int current_device_slot(int* dev_out) {
    int dev = 0;
    CMX_HIP(hipGetDevice(&dev));
    CMX_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal out of range");
    *dev_out = dev;
    return CMX_OK;
}

// Every kernel that needs more dynamic LDS than the default limit is listed here at load time (one entry per
// instantiation that a launch function names), so that cmx_init can raise all the limits up front and no first
// call has to -- hipFuncSetAttribute is not allowed while a stream is being captured into a graph.
struct LdsKernel {
    const void* fn;
    int bytes;
    PerDeviceFlag* flag;
};
std::vector<LdsKernel>& lds_registry() {
    static std::vector<LdsKernel> v;
    return v;
}
template <auto KFN, size_t SMEM>
struct LdsSetup {
    static inline PerDeviceFlag flag{};
    static inline const bool registered = (lds_registry().push_back({reinterpret_cast<const void*>(KFN), (int)SMEM, &flag}), true);
};

int allow_dynamic_lds(const void* kfn, int bytes, PerDeviceFlag& flag) {
    int dev = 0;
    int rc = current_device_slot(&dev);
    if (rc != CMX_OK) return rc;
    if (!flag.done[dev].load(std::memory_order_acquire)) {
        CMX_HIP(hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
        flag.done[dev].store(true, std::memory_order_release);
    }
    return CMX_OK;
}
// raises the limit of KFN on the current device unless cmx_init or an earlier call has done so
template <auto KFN, size_t SMEM>
int allow_dynamic_lds() {
    (void)LdsSetup<KFN, SMEM>::registered;
    return allow_dynamic_lds(reinterpret_cast<const void*>(KFN), (int)SMEM, LdsSetup<KFN, SMEM>::flag);
}

int cu_count(int* out) {
    static std::atomic<int> cus[kMaxDevices];
    int dev = 0;
    int rc = current_device_slot(&dev);
    if (rc != CMX_OK) return rc;
    int n = cus[dev].load(std::memory_order_acquire);
    if (n == 0) {
        CMX_HIP(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
        n = n > 0 ? n : 256;
        cus[dev].store(n, std::memory_order_release);
    }
    *out = n;
    return CMX_OK;
}

template <int FMT, int TW, int TM, int WW, int WM, int EPI, bool FAST>
int launch_gemm_impl(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    constexpr int kScaleDw = FMT == CMX_FMT_E2M1 ? 2 : 1;
    constexpr size_t smem = 2 * ((TW + TM) * kSlabBytes + (TW + TM) * 4 * kScaleDw);
    constexpr auto kfn = mx_gemm_kernel<FMT, TW, TM, WW, WM, EPI, FAST>;
    if (int rc = allow_dynamic_lds<kfn, smem>(); rc != CMX_OK) return rc;
    const uint64_t tiles = (uint64_t)max_m_tiles * p.w_tiles;
    CMX_REQUIRE(tiles > 0 && tiles < (1ull << 31), "tile count out of range");
    hipLaunchKernelGGL(kfn, dim3((uint32_t)tiles), dim3(64 * WW * WM), smem, s, p);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

template <int FMT, int TW, int TM, int WW, int WM, int EPI>
int launch_gemm_dl(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    constexpr int kScaleDw = FMT == CMX_FMT_E2M1 ? 2 : 1;
    constexpr size_t smem = 2 * (TW + TM) * kSlabBytes + 2 * (TW + TM) * kScaleDw * 4;
    constexpr auto kfn = mx_gemm_dl_kernel<FMT, TW, TM, WW, WM, EPI>;
    if (int rc = allow_dynamic_lds<kfn, smem>(); rc != CMX_OK) return rc;
    const uint64_t tiles = (uint64_t)max_m_tiles * p.w_tiles;
    CMX_REQUIRE(tiles > 0 && tiles < (1ull << 31), "tile count out of range");
    hipLaunchKernelGGL(kfn, dim3((uint32_t)tiles), dim3(64 * WW * WM), smem, s, p);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

template <int FMT, int EPI, int TM, int WW, int WM, int NSLOT>
int launch_gemm_pipe(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    // tile ring, scale ring (two-slot kernels: two blocks of 16 bytes per row), next-tile mailbox, 256-byte sink of the L2 prefetch loads
    // (+ the 16 KiB staging area of the whole-line stores, which overlays the last 512 bytes)
    constexpr size_t smem = NSLOT * (256 + TM) * kSlabBytes + (NSLOT == 2 ? 2 * (256 + TM) * 16 : NSLOT * (256 + TM) * 4) +
                            (pipe_stages_stores(NSLOT, EPI, WW, WM) ? 16384 : 512);
    constexpr auto kfn = mx_gemm_pipe_kernel<FMT, EPI, TM, WW, WM, NSLOT>;
    if (int rc = allow_dynamic_lds<kfn, smem>(); rc != CMX_OK) return rc;
    const uint64_t tiles = (uint64_t)max_m_tiles * p.w_tiles;
    CMX_REQUIRE(tiles > 0 && tiles < (1ull << 31), "tile count out of range");
    uint32_t grid = (uint32_t)tiles;
    if (pipe_is_persistent(NSLOT, EPI)) {
        // persistent: one workgroup per CU (the LDS footprint admits no second one), a multiple of the XCD count
        int cus = 0;
        if (int rc = cu_count(&cus); rc != CMX_OK) return rc;
        grid = (uint32_t)(cus / kXcds * kXcds);
        if (grid < (uint32_t)kXcds) grid = kXcds;
    }
    hipLaunchKernelGGL(kfn, dim3(grid), dim3(256), smem, s, p);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

template <int FMT, int EPI, int TM>
int launch_gemm_wreg(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    constexpr auto kfn = mx_gemm_wreg_kernel<FMT, EPI, TM>;
    constexpr size_t kWregLdsBytes = wreg_lds_bytes(TM);
    if (int rc = allow_dynamic_lds<kfn, kWregLdsBytes>(); rc != CMX_OK) return rc;
    const uint64_t tiles = (uint64_t)max_m_tiles * p.w_tiles;
    CMX_REQUIRE(tiles > 0 && tiles < (1ull << 31), "tile count out of range");
    // persistent: one workgroup per CU, a multiple of the XCD count
    int cus = 0;
    if (int rc = cu_count(&cus); rc != CMX_OK) return rc;
    uint32_t grid = (uint32_t)(cus / kXcds * kXcds);
    if (grid < (uint32_t)kXcds) grid = kXcds;
    hipLaunchKernelGGL(kfn, dim3(grid), dim3(256), kWregLdsBytes, s, p);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

template <int EPI, int WW, int WM>
int launch_gemm_pipe_fp4(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    // tile ring, ring of two scale blocks, next-tile mailbox and sink of the L2 prefetch loads (or the 16 KiB staging area of the
    // whole-line stores, which overlays those 512 bytes)
    constexpr size_t smem = 2 * 512 * kSlabBytes + 2 * 512 * 16 + (pipe_stages_stores(2, EPI, WW, WM) ? 16384 : 512);
    constexpr auto kfn = mx_gemm_pipe_fp4_kernel<EPI, WW, WM>;
    if (int rc = allow_dynamic_lds<kfn, smem>(); rc != CMX_OK) return rc;
    const uint64_t tiles = (uint64_t)max_m_tiles * p.w_tiles;
    CMX_REQUIRE(tiles > 0 && tiles < (1ull << 31), "tile count out of range");
    uint32_t grid = (uint32_t)tiles;
    if (pipe_is_persistent(2, EPI)) {
        // persistent: one workgroup per CU (the LDS footprint admits no second one), a multiple of the XCD count
        int cus = 0;
        if (int rc = cu_count(&cus); rc != CMX_OK) return rc;
        grid = (uint32_t)(cus / kXcds * kXcds);
        if (grid < (uint32_t)kXcds) grid = kXcds;
    }
    hipLaunchKernelGGL(kfn, dim3(grid), dim3(256), smem, s, p);
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

// The test build of this file (CMX_TEST_HOOKS, linked into the test library only) can force the register-staged
// kernels and pin the tile shape, so that tests reach every compiled instantiation; the product has neither switch.
#ifdef CMX_TEST_HOOKS
bool g_disable_dl = false;
#else
constexpr bool g_disable_dl = false;
#endif

template <int FMT, int TW, int TM, int WW, int WM, int EPI>
int launch_gemm(const GemmParams& p, uint32_t max_m_tiles, hipStream_t s) {
    // streaming kernel: whole 128-element scale groups, dword-aligned scale rows, four wavefronts
    if constexpr (TW % (8 * WW * WM) == 0 && TM % (8 * WW * WM) == 0 && TW % 64 == 0 && TM % 64 == 0) {
        if (!g_disable_dl && p.scale_vec && p.kbytes % kSlabBytes == 0)
            return launch_gemm_dl<FMT, TW, TM, WW, WM, EPI>(p, max_m_tiles, s);
    }
    const bool fast = p.scale_vec && (p.kbytes % kSlabBytes == 0);
    if (fast) return launch_gemm_impl<FMT, TW, TM, WW, WM, EPI, true>(p, max_m_tiles, s);
    return launch_gemm_impl<FMT, TW, TM, WW, WM, EPI, false>(p, max_m_tiles, s);
}

struct TileChoice {
    int tw, tm, waves;
};

#ifdef CMX_TEST_HOOKS
TileChoice g_force_tile = {0, 0, 0};   // tw == 0 -> heuristic
int g_pretiled_tile_rows = 0;          // 0 -> heuristic
#else
constexpr TileChoice g_force_tile = {0, 0, 0};
constexpr int g_pretiled_tile_rows = 0;
#endif

// waves: at 256 x 256 "4" and "5" select the hand-scheduled kernel in its 2 x 2 and 4 x 1 wavefront layouts
// when the problem is eligible for it (8-bit elements, whole 512-byte K blocks).  2 x 2 reads a fifth less
// from the LDS per slab and is the faster one on full tiles; grouped problems whose groups average less
// than two tiles of rows take 4 x 1, where every wavefront shares in whatever rows a ragged tile has
// (measured: 16 groups of ~2048 rows 891 vs 918 us in favour of 2 x 2, 256 groups of ~256 rows 4.33 vs
// 4.38 ms in favour of 4 x 1).  FP4 has its own hand-scheduled kernel in the same two layouts (K a multiple of 512
// elements; 16 groups of ~2048 rows at K = 7168, N = 4096: 2 x 2 persistent 565 us, one tile per workgroup 2 x 2
// 635 us and 4 x 1 700 us, the eight-wavefront streaming kernel, which takes every other FP4 problem, 750 us).
TileChoice choose_tile(uint32_t m_hint, uint32_t n, int fmt, bool grouped) {
    if (g_force_tile.tw) return g_force_tile;
    // short problems stream their weights once: the three-slot 256 x 128 kernel keeps two slabs in flight
    if (m_hint <= 128 && fmt != CMX_FMT_E2M1) return {256, 128, 5};
    if (m_hint <= 64) return {256, 64, 4};
    if (m_hint <= 128) return {256, 128, 8};
    return {256, 256, grouped && m_hint < 512 ? 5 : 4};
}

// Eight-wavefront shapes exist only as streaming kernels; when a problem is not eligible for
// streaming (ragged K, unaligned scale rows) the four-wavefront register-staged kernel of the same
// tile takes over.
template <int FMT, int TW, int TM, int EPI>
int launch_tile(const GemmParams& p, int waves, uint32_t max_m_tiles, hipStream_t s) {
    const bool stream_ok = !g_disable_dl && p.scale_vec && p.kbytes % kSlabBytes == 0;
    if constexpr (TW == 256 && TM == 256 && FMT != CMX_FMT_E2M1) {
        // whole four-slab scale blocks, fetched 16 bytes per row: K a multiple of 512 bytes, 16-byte aligned scale rows
        if ((waves == 4 || waves == 5) && stream_ok && p.scale_vec16 && p.kbytes % (4 * kSlabBytes) == 0) {
            // plain 16-bit output with 8-element-aligned rows takes the lean store epilogue and with it the persistent kernel
            constexpr int kLeanBf16 = EPI == kEpiStore ? kEpiStoreBf16 : EPI, kLeanFp16 = EPI == kEpiStore ? kEpiStoreFp16 : EPI;
            const bool lean = EPI == kEpiStore && p.out_type != CMX_OUT_FP32 && p.n % 8 == 0 && p.ldc % 8 == 0 &&
                              (reinterpret_cast<uintptr_t>(p.c) & 15u) == 0;
            // (the 4 x 1 layout with the lean store epilogue does not fit the register file without spilling
            // inside the loop, so the persistent store kernel is always 2 x 2)
            if (lean && p.out_type == CMX_OUT_BF16) return launch_gemm_pipe<FMT, kLeanBf16, 256, 2, 2, 2>(p, max_m_tiles, s);
            if (lean) return launch_gemm_pipe<FMT, kLeanFp16, 256, 2, 2, 2>(p, max_m_tiles, s);
            if (waves == 4) return launch_gemm_pipe<FMT, EPI, 256, 2, 2, 2>(p, max_m_tiles, s);
            return launch_gemm_pipe<FMT, EPI, 256, 4, 1, 2>(p, max_m_tiles, s);
        }
    }
    if constexpr (TW == 256 && TM == 256 && FMT == CMX_FMT_E2M1) {
        // hand-scheduled FP4 kernel: whole two-slab scale blocks (K a multiple of 512 elements), 16-byte aligned scale rows
        if ((waves == 4 || waves == 5) && stream_ok && p.scale_vec16 && p.kbytes % (2 * kSlabBytes) == 0) {
            if constexpr (EPI == kEpiStore) {
                // plain 16-bit output with 8-element-aligned rows: lean store epilogue, persistent kernel
                const bool lean = p.out_type != CMX_OUT_FP32 && p.n % 8 == 0 && p.ldc % 8 == 0 && (reinterpret_cast<uintptr_t>(p.c) & 15u) == 0;
                // (unlike the 8-bit kernel, whose fragments take twice the registers, the 4 x 1 layout fits here too)
                if (lean && waves == 4 && p.out_type == CMX_OUT_BF16) return launch_gemm_pipe_fp4<kEpiStoreBf16, 2, 2>(p, max_m_tiles, s);
                if (lean && waves == 4) return launch_gemm_pipe_fp4<kEpiStoreFp16, 2, 2>(p, max_m_tiles, s);
                if (lean && p.out_type == CMX_OUT_BF16) return launch_gemm_pipe_fp4<kEpiStoreBf16, 4, 1>(p, max_m_tiles, s);
                if (lean) return launch_gemm_pipe_fp4<kEpiStoreFp16, 4, 1>(p, max_m_tiles, s);
                if (waves == 4) return launch_gemm_pipe_fp4<EPI, 2, 2>(p, max_m_tiles, s);
                return launch_gemm_pipe_fp4<EPI, 4, 1>(p, max_m_tiles, s);
            }
        }
    }
    if constexpr (TW == 256 && TM == 128 && FMT != CMX_FMT_E2M1) {
        if (waves == 5 && stream_ok) return launch_gemm_pipe<FMT, EPI, 128, 4, 1, 3>(p, max_m_tiles, s);
    }
    if constexpr (TM >= 128) {
        // the four-wavefront streaming kernel of the 256 x 256 tile runs out of registers: eight there
        if ((waves == 8 || (TW == 256 && TM == 256)) && stream_ok) return launch_gemm_dl<FMT, TW, TM, 2, 4, EPI>(p, max_m_tiles, s);
    }
    constexpr int WW = TM >= 128 ? 2 : 4, WM = TM >= 128 ? 2 : 1;
    return launch_gemm<FMT, TW, TM, WW, WM, EPI>(p, max_m_tiles, s);
}

template <int FMT, int EPI>
int dispatch_tile(const GemmParams& p, TileChoice t, uint32_t max_m_tiles, hipStream_t s) {
    if (t.tw == 256 && t.tm == 256) return launch_tile<FMT, 256, 256, EPI>(p, t.waves, max_m_tiles, s);
    if (t.tw == 256 && t.tm == 128) return launch_tile<FMT, 256, 128, EPI>(p, t.waves, max_m_tiles, s);
    if (t.tw == 256 && t.tm == 64) return launch_tile<FMT, 256, 64, EPI>(p, t.waves, max_m_tiles, s);
    if (t.tw == 128 && t.tm == 128) return launch_tile<FMT, 128, 128, EPI>(p, t.waves, max_m_tiles, s);
    set_error("unsupported tile shape");
    return CMX_EINVAL;
}

// Pre-tiled weights (cmx_mx_pretile_weights): only the weights-to-registers kernel reads that order, so a problem it
// cannot take is an error, not a reason to fall back.
int check_pretiled(const GemmParams& p, int fmt, bool swiglu) {
    CMX_REQUIRE(fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2, "pre-tiled weights: 8-bit element formats only");
    CMX_REQUIRE(p.kbytes % (4 * kSlabBytes) == 0, "pre-tiled weights: k must be a multiple of 512");
    CMX_REQUIRE(p.scale_vec16, "pre-tiled weights: scale rows of both operands must be 16-byte aligned");
    // (with the bf16 activation output on top, the SwiGLU epilogue no longer fits the register file beside the weight ring)
    CMX_REQUIRE(!swiglu || p.act_bf16 == nullptr, "pre-tiled weights: no bf16 activation output (act_bf16 must be NULL)");
    CMX_REQUIRE(swiglu || (p.out_type != CMX_OUT_FP32 && p.n % 8 == 0 && p.ldc % 8 == 0 && (reinterpret_cast<uintptr_t>(p.c) & 15u) == 0),
                "pre-tiled weights: 16-bit output, n and ldc multiples of 8, c 16-byte aligned");
    return CMX_OK;
}

template <int TM>
int launch_pretiled(const GemmParams& p, int fmt, bool swiglu, uint32_t max_m_tiles, hipStream_t s) {
    if (swiglu) return launch_gemm_wreg<CMX_FMT_E4M3, kEpiSwigluQuant, TM>(p, max_m_tiles, s);
    if (fmt == CMX_FMT_E4M3) {
        if (p.out_type == CMX_OUT_BF16) return launch_gemm_wreg<CMX_FMT_E4M3, kEpiStoreBf16, TM>(p, max_m_tiles, s);
        return launch_gemm_wreg<CMX_FMT_E4M3, kEpiStoreFp16, TM>(p, max_m_tiles, s);
    }
    if (p.out_type == CMX_OUT_BF16) return launch_gemm_wreg<CMX_FMT_E5M2, kEpiStoreBf16, TM>(p, max_m_tiles, s);
    return launch_gemm_wreg<CMX_FMT_E5M2, kEpiStoreFp16, TM>(p, max_m_tiles, s);
}

int check_operands(const void* a, uint32_t lda, const void* as, uint32_t ld_as, const void* w, uint32_t ldw,
                   const void* ws, uint32_t ld_ws, uint32_t k, int fmt) {
    CMX_REQUIRE(a && as && w && ws, "null pointer");
    CMX_REQUIRE(fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2 || fmt == CMX_FMT_E2M1, "unknown element format");
    CMX_REQUIRE(k > 0 && k % 32 == 0, "k must be a positive multiple of 32");
    const uint32_t kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k;
    CMX_REQUIRE(lda >= kbytes && ldw >= kbytes, "operand row pitch smaller than a row");
    CMX_REQUIRE(lda % 16 == 0 && ldw % 16 == 0 && aligned16(a) && aligned16(w), "operand rows must be 16-byte aligned");
    CMX_REQUIRE(ld_as >= k / 32 && ld_ws >= k / 32, "scale row pitch smaller than a row");
    return CMX_OK;
}

bool scales_aligned16(const void* as, uint32_t ld_as, const void* ws, uint32_t ld_ws) {
    return ld_as % 16 == 0 && ld_ws % 16 == 0 && (reinterpret_cast<uintptr_t>(as) & 15u) == 0 &&
           (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
}

bool scales_dword_aligned(const void* as, uint32_t ld_as, const void* ws, uint32_t ld_ws) {
    return ld_as % 4 == 0 && ld_ws % 4 == 0 && (reinterpret_cast<uintptr_t>(as) & 3u) == 0 &&
           (reinterpret_cast<uintptr_t>(ws) & 3u) == 0;
}

}  // namespace

}  // namespace cmx

#ifdef CMX_TEST_HOOKS
extern "C" int cmx_debug_disable_streaming(int off) {
    cmx::g_disable_dl = off != 0;
    return CMX_OK;
}

// pin the tile height (256 or 288 rows) of every later matmul call on pre-tiled weights (0 restores the heuristic)
extern "C" int cmx_debug_pretiled_tile_rows(int rows) {
    cmx::g_pretiled_tile_rows = rows == 256 || rows == 288 ? rows : 0;
    return CMX_OK;
}

// pin the tile shape and wavefront count of every later matmul call (tw = 0 restores the heuristic)
extern "C" int cmx_debug_force_tile(int tw, int tm, int waves) {
    cmx::g_force_tile = (tw > 0 && tm > 0) ? cmx::TileChoice{tw, tm, waves > 0 ? waves : 4} : cmx::TileChoice{0, 0, 0};
    return CMX_OK;
}
#endif

extern "C" int cmx_mx_gemm(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b,
                           uint32_t ldb, const uint8_t* b_scale, uint32_t ld_bs, void* c, uint32_t ldc, uint32_t m,
                           uint32_t n, uint32_t k, int fmt, int out_type, cmx_stream_t stream) {
    using namespace cmx;
    if (m == 0 || n == 0) return CMX_OK;
    int rc = check_operands(a, lda, a_scale, ld_as, b, ldb, b_scale, ld_bs, k, fmt);
    if (rc != CMX_OK) return rc;
    CMX_REQUIRE(c && ldc >= n, "bad output");
    CMX_REQUIRE(out_type == CMX_OUT_BF16 || out_type == CMX_OUT_FP16 || out_type == CMX_OUT_FP32, "unknown output type");
    GemmParams p{};
    p.a = a; p.a_scale = a_scale; p.w = b; p.w_scale = b_scale; p.c = c;
    p.lda = lda; p.ld_as = ld_as; p.ldw = ldb; p.ld_ws = ld_bs; p.ldc = ldc;
    p.m = m; p.n = n; p.kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k; p.kblocks = k / 32;
    p.groups = 1; p.out_type = out_type;
    p.scale_vec = scales_dword_aligned(a_scale, ld_as, b_scale, ld_bs);
    p.scale_vec16 = scales_aligned16(a_scale, ld_as, b_scale, ld_bs);
    CMX_REQUIRE((uint64_t)n * ldb < (1ull << 32) && (uint64_t)lda * 256 < (1ull << 32), "operand tile exceeds 32-bit offsets");
    TileChoice t = choose_tile(m, n, fmt, false);
    p.w_tiles = ceil_div(n, t.tw);
    const uint32_t m_tiles = ceil_div(m, t.tm);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (fmt) {
        case CMX_FMT_E4M3: return dispatch_tile<CMX_FMT_E4M3, kEpiStore>(p, t, m_tiles, s);
        case CMX_FMT_E5M2: return dispatch_tile<CMX_FMT_E5M2, kEpiStore>(p, t, m_tiles, s);
        default: return dispatch_tile<CMX_FMT_E2M1, kEpiStore>(p, t, m_tiles, s);
    }
}

extern "C" size_t cmx_mx_gmm_workspace_bytes(uint32_t groups) {
    // row offsets, m-tile prefix, per-XCD tile counters
    return cmx::round_up_sz((2 * (size_t)(groups + 1) + 8) * sizeof(int32_t), 256);
}

namespace cmx {
namespace {
int gmm_common(GemmParams& p, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, void* workspace, int fmt,
               bool swiglu, hipStream_t s) {
    CMX_REQUIRE(group_sizes && workspace, "null pointer");
    CMX_REQUIRE(groups > 0 && groups <= 65536, "bad group count");
    CMX_REQUIRE(m_total < (1u << 31), "too many rows");
    CMX_REQUIRE((uint64_t)p.n * p.ldw < (1ull << 32) && (uint64_t)p.lda * 256 < (1ull << 32),
                "operand tile exceeds 32-bit offsets");
    CMX_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 3u) == 0, "workspace must be 4-byte aligned");
    if (p.w_pretiled)
        if (int rc = check_pretiled(p, fmt, swiglu); rc != CMX_OK) return rc;
    // average rows per group steers the tile height
    TileChoice t = choose_tile(ceil_div(m_total, groups), p.n, fmt, true);
    // the weights-to-registers kernel, tiles drawn from the counters: 256 x 288 when the groups average less than four
    // tiles of rows (a group of 257 to 288 rows then takes one pass over its weights instead of two), else 256 x 256
    if (p.w_pretiled) t = {256, g_pretiled_tile_rows ? g_pretiled_tile_rows : (ceil_div(m_total, groups) < 1024 ? 288 : 256), 5};
    int32_t* row_off = static_cast<int32_t*>(workspace);
    int32_t* tile_pref = row_off + (groups + 1);
    int32_t* tile_ctr = tile_pref + (groups + 1);
    hipLaunchKernelGGL(gmm_prepare_kernel, dim3(1), dim3(256), 0, s, group_sizes, groups, (uint32_t)t.tm, m_total, row_off,
                       tile_pref, tile_ctr);
    CMX_LAUNCH_CHECK();
    p.row_off = row_off;
    p.tile_pref = tile_pref;
    // The persistent kernels draw their next tile from a per-XCD counter when tiles differ in cost (4 x 1 wavefronts skip
    // the MFMAs of absent rows).  With 2 x 2 wavefronts every tile costs the same, so those kernels walk their XCD's run in
    // fixed strides instead: no atomic whose result has to be waited for with everything else in flight.
    p.tile_ctr = t.waves == 4 ? nullptr : tile_ctr;
    p.groups = groups;
    p.w_tiles = swiglu ? ceil_div(p.n / 2, t.tw / 2) : ceil_div(p.n, t.tw);
    const uint32_t max_m_tiles = m_total / t.tm + groups;
    if (p.w_pretiled) return t.tm == 288 ? launch_pretiled<288>(p, fmt, swiglu, max_m_tiles, s) : launch_pretiled<256>(p, fmt, swiglu, max_m_tiles, s);
    if (swiglu && p.act_bf16 != nullptr) return dispatch_tile<CMX_FMT_E4M3, kEpiSwigluQuantAct>(p, t, max_m_tiles, s);
    if (swiglu) return dispatch_tile<CMX_FMT_E4M3, kEpiSwigluQuant>(p, t, max_m_tiles, s);
    switch (fmt) {
        case CMX_FMT_E4M3: return dispatch_tile<CMX_FMT_E4M3, kEpiStore>(p, t, max_m_tiles, s);
        case CMX_FMT_E5M2: return dispatch_tile<CMX_FMT_E5M2, kEpiStore>(p, t, max_m_tiles, s);
        default: return dispatch_tile<CMX_FMT_E2M1, kEpiStore>(p, t, max_m_tiles, s);
    }
}
}  // namespace
}  // namespace cmx

namespace cmx {
namespace {
int gmm_store(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b, const uint8_t* b_scale,
              void* c, uint32_t ldc, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n, uint32_t k,
              int fmt, int out_type, void* workspace, bool pretiled, cmx_stream_t stream) {
    if (m_total == 0 || n == 0) return CMX_OK;
    const uint32_t kbytes = fmt == CMX_FMT_E2M1 ? k / 2 : k;
    // weight scale rows are as every producer writes them: padded to an even count (the quantizer, the
    // reference generator's transposed even-padded matrix, the host operators' ScaleCols(k))
    const uint32_t ld_ws = scale_cols(k);
    int rc = check_operands(a, lda, a_scale, ld_as, b, kbytes, b_scale, ld_ws, k, fmt);
    if (rc != CMX_OK) return rc;
    CMX_REQUIRE(c && ldc >= n, "bad output");
    CMX_REQUIRE(out_type == CMX_OUT_BF16 || out_type == CMX_OUT_FP16 || out_type == CMX_OUT_FP32, "unknown output type");
    GemmParams p{};
    p.a = a; p.a_scale = a_scale; p.w = b; p.w_scale = b_scale; p.c = c;
    p.lda = lda; p.ld_as = ld_as; p.ldw = kbytes; p.ld_ws = ld_ws; p.ldc = ldc;
    p.m = m_total; p.n = n; p.kbytes = kbytes; p.kblocks = k / 32; p.out_type = out_type;
    p.scale_vec = scales_dword_aligned(a_scale, ld_as, b_scale, ld_ws);
    p.scale_vec16 = scales_aligned16(a_scale, ld_as, b_scale, ld_ws);
    p.w_pretiled = pretiled ? 1 : 0;
    return gmm_common(p, group_sizes, groups, m_total, workspace, fmt, false, static_cast<hipStream_t>(stream));
}
}  // namespace
}  // namespace cmx

extern "C" int cmx_mx_gmm(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b,
                          const uint8_t* b_scale, void* c, uint32_t ldc, const int32_t* group_sizes, uint32_t groups,
                          uint32_t m_total, uint32_t n, uint32_t k, int fmt, int out_type, void* workspace,
                          cmx_stream_t stream) {
    return cmx::gmm_store(a, lda, a_scale, ld_as, b, b_scale, c, ldc, group_sizes, groups, m_total, n, k, fmt, out_type,
                          workspace, false, stream);
}

extern "C" int cmx_mx_gmm_pretiled(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                   const uint8_t* b_tiled, const uint8_t* b_scale, void* c, uint32_t ldc,
                                   const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n, uint32_t k,
                                   int fmt, int out_type, void* workspace, cmx_stream_t stream) {
    return cmx::gmm_store(a, lda, a_scale, ld_as, b_tiled, b_scale, c, ldc, group_sizes, groups, m_total, n, k, fmt,
                          out_type, workspace, true, stream);
}

extern "C" size_t cmx_int8_gmm_workspace_bytes(uint32_t groups, uint32_t n, uint32_t k, int trans_b) {
    const size_t meta = cmx::round_up_sz(cmx_mx_gmm_workspace_bytes(groups), 256);
    return meta + (trans_b ? 0 : cmx::round_up_sz((size_t)groups * n * k, 256));
}

extern "C" int cmx_int8_gmm_dequant_swiglu(const int8_t* a, uint32_t lda, const float* token_scale, const int8_t* b,
                                           const float* channel_scale, uint32_t channel_scale_stride, void* out,
                                           uint32_t ld_out, int out_type, const int32_t* group_sizes, uint32_t groups,
                                           uint32_t m_total, uint32_t n, uint32_t k, int trans_b, void* workspace,
                                           cmx_stream_t stream) {
    using namespace cmx;
    if (m_total == 0 || n == 0) return CMX_OK;
    CMX_REQUIRE(a && token_scale && b && channel_scale && out && group_sizes && workspace, "null pointer");
    CMX_REQUIRE(groups > 0 && groups <= 65536 && m_total < (1u << 31), "bad group count or too many rows");
    CMX_REQUIRE(k > 0 && k % kSlabBytes == 0 && k < (1u << 17), "k must be a multiple of 128 below 131072 (INT32 accumulation)");
    CMX_REQUIRE(n % 64 == 0, "n must be a multiple of 64 (32-wide gate and up fragments)");
    CMX_REQUIRE(lda >= k && lda % 16 == 0 && aligned16(a) && aligned16(b), "operand rows must be 16-byte aligned");
    CMX_REQUIRE(ld_out >= n / 2 && channel_scale_stride >= 1, "bad output pitch or scale stride");
    CMX_REQUIRE(out_type == CMX_OUT_BF16 || out_type == CMX_OUT_FP16 || out_type == CMX_OUT_FP32, "unknown output type");
    CMX_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "workspace must be 256-byte aligned");
    CMX_REQUIRE((uint64_t)n * k < (1ull << 32) && (uint64_t)lda * 256 < (1ull << 32), "operand tile exceeds 32-bit offsets");
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    const uint8_t* w = reinterpret_cast<const uint8_t*>(b);
    if (!trans_b) {
        // weights stored [groups, k, n]: rewrite them K-contiguous behind the schedule metadata
        uint8_t* wt = ws + round_up_sz(cmx_mx_gmm_workspace_bytes(groups), 256);
        int rc = cmx_bytes_to_k_major(w, n, wt, k, k, n, groups, stream);
        if (rc != CMX_OK) return rc;
        w = wt;
    }
    GemmParams p{};
    p.a = reinterpret_cast<const uint8_t*>(a);
    p.a_scale = reinterpret_cast<const uint8_t*>(token_scale);
    p.w = w;
    p.w_scale = reinterpret_cast<const uint8_t*>(channel_scale);
    p.c = out;
    p.lda = lda; p.ld_as = 0; p.ldw = k; p.ld_ws = channel_scale_stride; p.ldc = ld_out;
    p.m = m_total; p.n = n; p.kbytes = k; p.kblocks = k / 32; p.out_type = out_type;
    p.scale_vec = 1;
    int32_t* row_off = reinterpret_cast<int32_t*>(ws);
    int32_t* tile_pref = row_off + (groups + 1);
    int32_t* tile_ctr = tile_pref + (groups + 1);
    constexpr int kTile = 256;
    hipLaunchKernelGGL(gmm_prepare_kernel, dim3(1), dim3(256), 0, s, group_sizes, groups, (uint32_t)kTile, m_total, row_off,
                       tile_pref, tile_ctr);
    CMX_LAUNCH_CHECK();
    p.row_off = row_off;
    p.tile_pref = tile_pref;
    p.tile_ctr = tile_ctr;
    p.groups = groups;
    p.w_tiles = ceil_div(n / 2, kTile / 2);
    // (hand-scheduled variants of this kernel were measured twice at 16 x 2048 x 7168 x 4096 and are not kept: two i8
    // MFMAs per step and accumulator in the 8-bit schedule 997 us, one per 32-K step in the 16-byte-fragment
    // schedule shared with FP4, one tile per workgroup, 994-1000 us, against 967-975 us for this one)
    return launch_gemm_dl<kFmtI8, kTile, kTile, 2, 4, kEpiI8DequantSwiglu>(p, m_total / kTile + groups, s);
}

namespace cmx {
namespace {
int gmm_swiglu_quant(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as, const uint8_t* b,
                     const uint8_t* b_scale, uint8_t* act_codes, uint32_t ld_act, uint8_t* act_scales, uint32_t ld_acts,
                     void* act_bf16, const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n, uint32_t k,
                     void* workspace, bool pretiled, cmx_stream_t stream) {
    const uint32_t ld_ws = scale_cols(k);      // even-padded weight scale rows, as in cmx_mx_gmm
    int rc = check_operands(a, lda, a_scale, ld_as, b, k, b_scale, ld_ws, k, CMX_FMT_E4M3);
    if (rc != CMX_OK) return rc;
    CMX_REQUIRE(n % 64 == 0, "n must be a multiple of 64 (gate|up halves of whole MX blocks)");
    CMX_REQUIRE(act_codes && act_scales, "null pointer");
    CMX_REQUIRE(ld_act >= n / 2 && ld_act % 4 == 0 && (reinterpret_cast<uintptr_t>(act_codes) & 3u) == 0,
                "activation code rows must be 4-byte aligned and hold n/2 bytes");
    CMX_REQUIRE(ld_acts >= scale_cols(n / 2), "activation scale pitch too small");
    GemmParams p{};
    p.a = a; p.a_scale = a_scale; p.w = b; p.w_scale = b_scale;
    p.act_codes = act_codes; p.act_scales = act_scales; p.act_bf16 = static_cast<uint16_t*>(act_bf16);
    p.ld_act = ld_act; p.ld_acts = ld_acts;
    p.lda = lda; p.ld_as = ld_as; p.ldw = k; p.ld_ws = ld_ws;
    p.m = m_total; p.n = n; p.kbytes = k; p.kblocks = k / 32; p.out_type = CMX_OUT_BF16;
    p.scale_vec = scales_dword_aligned(a_scale, ld_as, b_scale, ld_ws);
    p.scale_vec16 = scales_aligned16(a_scale, ld_as, b_scale, ld_ws);
    p.w_pretiled = pretiled ? 1 : 0;
    return gmm_common(p, group_sizes, groups, m_total, workspace, CMX_FMT_E4M3, true, static_cast<hipStream_t>(stream));
}

// Schedule metadata of the allocation-free entry point (row offsets, m-tile prefix, per-XCD tile counters of up to
// kStaticGroups groups): a fixed array in device memory instead of a caller's workspace.  Every device that runs
// the library holds its own copy; its address on a device comes from hipGetSymbolAddress with that device current
// (the array's name is only a host-side handle).
constexpr uint32_t kStaticGroups = 4096;
constexpr size_t kStaticScratchBytes = (2 * ((size_t)kStaticGroups + 1) + 8) * sizeof(int32_t);
static __device__ __align__(256) unsigned char scratch[(kStaticScratchBytes + 255) / 256 * 256];

int static_scratch(void** out) {
    static std::atomic<void*> ptrs[kMaxDevices];
    int dev = 0;
    int rc = current_device_slot(&dev);
    if (rc != CMX_OK) return rc;
    void* q = ptrs[dev].load(std::memory_order_acquire);
    if (q == nullptr) {
        CMX_HIP(hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)));
        CMX_REQUIRE(q != nullptr, "no device address for the static scratch array");
        ptrs[dev].store(q, std::memory_order_release);
    }
    *out = q;
    return CMX_OK;
}
}  // namespace
}  // namespace cmx

extern "C" int cmx_mx_gmm_swiglu_quant(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                       const uint8_t* b, const uint8_t* b_scale, uint8_t* act_codes, uint32_t ld_act,
                                       uint8_t* act_scales, uint32_t ld_acts, void* act_bf16,
                                       const int32_t* group_sizes, uint32_t groups, uint32_t m_total, uint32_t n,
                                       uint32_t k, void* workspace, cmx_stream_t stream) {
    if (m_total == 0 || n == 0) return CMX_OK;
    return cmx::gmm_swiglu_quant(a, lda, a_scale, ld_as, b, b_scale, act_codes, ld_act, act_scales, ld_acts, act_bf16,
                                 group_sizes, groups, m_total, n, k, workspace, false, stream);
}

extern "C" int cmx_mx_gmm_swiglu_quant_pretiled(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                                const uint8_t* b_tiled, const uint8_t* b_scale, uint8_t* act_codes,
                                                uint32_t ld_act, uint8_t* act_scales, uint32_t ld_acts, void* act_bf16,
                                                const int32_t* group_sizes, uint32_t groups, uint32_t m_total,
                                                uint32_t n, uint32_t k, void* workspace, cmx_stream_t stream) {
    if (m_total == 0 || n == 0) return CMX_OK;
    return cmx::gmm_swiglu_quant(a, lda, a_scale, ld_as, b_tiled, b_scale, act_codes, ld_act, act_scales, ld_acts,
                                 act_bf16, group_sizes, groups, m_total, n, k, workspace, true, stream);
}

extern "C" uint32_t cmx_mx_gmm_noalloc_max_groups(void) { return cmx::kStaticGroups; }

extern "C" int cmx_mx_gmm_swiglu_quant_noalloc(const uint8_t* a, uint32_t lda, const uint8_t* a_scale, uint32_t ld_as,
                                               const uint8_t* b, const uint8_t* b_scale, uint8_t* act_codes,
                                               uint32_t ld_act, uint8_t* act_scales, uint32_t ld_acts, void* act_bf16,
                                               const int32_t* group_sizes, uint32_t groups, uint32_t m_total,
                                               uint32_t n, uint32_t k, cmx_stream_t stream) {
    using namespace cmx;
    if (m_total == 0 || n == 0) return CMX_OK;
    CMX_REQUIRE(groups <= kStaticGroups, "at most 4096 groups fit the static schedule array: use cmx_mx_gmm_swiglu_quant with a workspace");
    void* meta = nullptr;
    if (int rc = static_scratch(&meta); rc != CMX_OK) return rc;
    // gmm_prepare_kernel rewrites every word of the metadata that the matmul kernel reads (and zeroes the tile
    // counters), so nothing of an earlier call survives into this one
    return gmm_swiglu_quant(a, lda, a_scale, ld_as, b, b_scale, act_codes, ld_act, act_scales, ld_acts, act_bf16,
                            group_sizes, groups, m_total, n, k, meta, false, stream);
}

// One-time set-up on the current device: raises the dynamic-LDS limit of every matmul kernel, has the runtime load the
// code object of every translation unit, reads the CU count and resolves the static schedule array, so that no later
// call has to (none of this is allowed, or wise, inside a stream capture).  Optional: every entry point still does
// what it needs on first use.
extern "C" int cmx_init(void) {
    using namespace cmx;
    for (const LdsKernel& k : lds_registry())
        if (int rc = allow_dynamic_lds(k.fn, k.bytes, *k.flag); rc != CMX_OK) return rc;
    // the matmul kernels without an LDS limit to raise (and with them this unit's code object), then the other units
    hipFuncAttributes attr;
    CMX_HIP(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(gmm_prepare_kernel)));
    if (int rc = preload_routing_kernels(); rc != CMX_OK) return rc;
    if (int rc = preload_layout_kernels(); rc != CMX_OK) return rc;
    if (int rc = preload_quant_kernels(); rc != CMX_OK) return rc;
    int cus = 0;
    if (int rc = cu_count(&cus); rc != CMX_OK) return rc;
    void* meta = nullptr;
    return static_scratch(&meta);
}
