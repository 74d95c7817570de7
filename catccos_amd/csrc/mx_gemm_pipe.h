// Hand-scheduled 256 x 256 block-scaled matmul kernel for the 8-bit MX formats (included by
// mx_gemm.hip inside its namespace).
//
// Four wavefronts, one per SIMD, each owning a 128 x 128 corner of the tile: 16 accumulator tiles
// (256 AGPRs) and two sets of 8 operand fragments (128 VGPRs).  With a single wavefront per SIMD the
// matrix pipe only stays busy if the instruction stream itself interleaves the LDS reads and the
// LDS-DMA loads between the MFMAs, and if nothing waits on a load it has just issued.  The compiler's
// scheduler clusters such loads and waits for them at once, so the steady-state loop is written as
// a fixed sequence of single-instruction asm statements (their order is kept) with hand-placed
// s_waitcnt; the compiler still allocates the registers.
//
// One slab = 128 bytes of K = two MFMA steps.  Per slab and wavefront:
//   step 0: 16 MFMAs on fragment set 0; behind the first 8, the 16 reads of fragment set 1 (second
//           half of the slab); then wait for the own loads of slab s+1 and the own reads of slab s,
//           barrier (slot s is now free and slab s+1 is visible to everyone);
//   step 1: 16 MFMAs on fragment set 1; behind them the 16+2 LDS-DMA loads of slab s+2 into the
//           freed slot, the 16 reads of fragment set 0 from slab s+1 and its 8 scale dwords.
// Every LDS address is a per-lane base register plus an immediate, every global address a per-lane
// offset register plus a scalar slab offset: the loop contains no address arithmetic on the VALU.
#pragma once

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int OFF>
__device__ __forceinline__ v4i lds_read_b128(uint32_t addr) {
    v4i r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
template <int OFF>
__device__ __forceinline__ uint32_t lds_read_b32(uint32_t addr) {
    uint32_t r;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
__device__ __forceinline__ void dma_b128(uint32_t lds_dst, uint32_t voff, v4i rsrc, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}
__device__ __forceinline__ void dma_b32(uint32_t lds_dst, uint32_t voff, v4i rsrc, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}

// acc += W-fragment x A-fragment with the scale byte pair SEL (0: bytes 0/1 of the slab's dword by
// half-wave, 2: bytes 2/3) of the shifted scale registers.
template <int FMT, int SEL>
__device__ __forceinline__ void mfma_acc(v16f& acc, const v8i& w, const v8i& a, uint32_t sw, uint32_t sa) {
    static_assert(SEL == 0 || SEL == 2, "scale byte pair");
    if constexpr (FMT == CMX_FMT_E4M3) {
        if constexpr (SEL == 0)
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
        else
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[1,1,0]"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
    } else {
        if constexpr (SEL == 0)
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:1 blgp:1"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
        else
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[1,1,0] cbsz:1 blgp:1"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
    }
}

// Order in which the 8 fragments (0-3 weights, 4-7 activations) are read = order of first use by the
// MFMA sequence (weight fragment outer, activation fragment inner).
__device__ __forceinline__ constexpr int pipe_read_order(int i) {
    return i == 0 ? 0 : (i <= 4 ? 3 + i : i - 4);
}

__device__ __forceinline__ v8i join8(const v4i& lo, const v4i& hi) {
    return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

template <int FMT, int EPI>
__global__ __launch_bounds__(256) void mx_gemm_pipe_kernel(const GemmParams p) {
    static_assert(FMT == CMX_FMT_E4M3 || FMT == CMX_FMT_E5M2, "8-bit element formats only");
    constexpr int TW = 256, TM = 256, WW = 2, WM = 2, NW = 4, FW = 4, FM = 4;
    constexpr int kRows = TW + TM;
    constexpr int kSlotBytes = kRows * kSlabBytes;            // 64 KiB
    constexpr int kScaleBase = 2 * kSlotBytes;                // scale ring behind the two tile slots
    constexpr int kScaleSlotBytes = kRows * 4;
    constexpr int kTileLoads = kRows / (8 * NW);              // 16 LDS-DMA loads per wavefront and slab
    constexpr int kWTileLoads = TW / (8 * NW);                // the first 8 fetch weight rows

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

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

#ifndef CMX_PIPE_DBG
#define CMX_PIPE_DBG 0
#endif
    const uint8_t* wg = p.w + (size_t)g * p.n * p.ldw;
    const uint8_t* wsg = p.w_scale + (size_t)g * p.n * p.ld_ws;
    const uint8_t* ag = p.a + (size_t)row0 * p.lda;
    const uint8_t* asg = p.a_scale + (size_t)row0 * p.ld_as;

    // global row of tile row r (rows past the edge re-read the last valid row; their results are never stored)
    auto wrow_of = [&](uint32_t r) -> uint32_t {
        uint32_t gr;
        if (EPI == kEpiSwigluQuant) {
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

    // ---- LDS-DMA: per-lane global offsets (constant over K) ---------------------------------------
    // load i of this wavefront fills combined tile rows (4i + wave)*8 .. +8; lane q -> row +q/8, LDS
    // chunk q%8, and fetches the global chunk that the XOR swizzle maps there
    uint32_t goff[kTileLoads];
#pragma unroll
    for (int i = 0; i < kTileLoads; ++i) {
        const uint32_t cr = (NW * i + wave) * 8 + (lane >> 3);
        const uint32_t logical = swz(cr, lane & 7u);
        goff[i] = (i < kWTileLoads ? wrow_of(cr) * p.ldw : arow_of(cr - TW) * p.lda) + logical * 16;
        if (CMX_PIPE_DBG & 2) goff[i] = (i < kWTileLoads ? (cr - wt * 0) * p.ldw : (cr - TW) * p.lda) + logical * 16;
    }
    // scale dwords: this wavefront fetches those of weight rows 64*wave.. and activation rows 64*wave..
    const uint32_t sgoff_w = wrow_of(64 * wave + lane) * p.ld_ws;
    const uint32_t sgoff_a = arow_of(64 * wave + lane) * p.ld_as;

    auto make_rsrc = [](const uint8_t* q) -> v4i {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        v4i r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));     // stride 0
        r[2] = -1;                                                           // no range limit
        r[3] = 0x00020000;
        return r;
    };
    const v4i w_rs = make_rsrc((CMX_PIPE_DBG & 2) ? p.w : wg), a_rs = make_rsrc((CMX_PIPE_DBG & 2) ? p.a : ag), ws_rs = make_rsrc(wsg), as_rs = make_rsrc(asg);

    const uint32_t nslab = p.kbytes / kSlabBytes;
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sdma_base = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + wave * 256);

    auto issue_tile_load = [&](int slot, int i, uint32_t koff) {
        dma_b128(dma_base + slot * kSlotBytes + i * (NW * 1024), goff[i], i < kWTileLoads ? w_rs : a_rs, koff);
    };
    auto issue_scale_loads = [&](int slot, uint32_t soff) {
        dma_b32(sdma_base + slot * kScaleSlotBytes, sgoff_w, ws_rs, soff);
        dma_b32(sdma_base + slot * kScaleSlotBytes + TW * 4, sgoff_a, as_rs, soff);
    };
    auto clamp_slab = [&](uint32_t slab) -> uint32_t { return slab < nslab ? slab : nslab - 1; };   // past the end: harmless reload

    // ---- fragment read addresses ------------------------------------------------------------------
    // a lane reads 16-byte chunks lh, lh+2 (step 0) and lh+4, lh+6 (step 1) of its row; all rows of a
    // lane share the low five bits l32, hence the swizzle term
    const uint32_t x = (l32 & 7u) ^ ((l32 >> 3) & 1u);
    const uint32_t w_row_base = EPI == kEpiSwigluQuant ? ww * (TW / 2 / WW) : ww * (TW / WW);
    uint32_t wb[2][4], ab[2][4];       // [slot][chunk j]
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t ch = ((lh + 2 * j) ^ x) * 16;
            wb[s][j] = lds0 + s * kSlotBytes + (w_row_base + l32) * kSlabBytes + ch;
            ab[s][j] = lds0 + s * kSlotBytes + (TW + wm * (TM / WM) + l32) * kSlabBytes + ch;
        }
    const uint32_t swb = lds0 + kScaleBase + (w_row_base + l32) * 4;
    const uint32_t sab = lds0 + kScaleBase + (TW + wm * (TM / WM) + l32) * 4;
    const uint32_t sshift = 8 * lh;

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // fragment sets: index 0..3 weights, 4..7 activations; lo = registers 0-3, hi = registers 4-7
    v4i f0lo[8], f0hi[8], f1lo[8], f1hi[8];
    uint32_t sraw[8], scur[2][8];      // shifted scales alternate between two sets: a set is rewritten one slab after its last use

    // weight fragment f sits f*32 rows (SwiGLU: gate fragments 0,1 then their up partners 128 rows on) below the base
    // read order = order of first use by the MFMA sequence (fw outer, fm inner): W0 A0 A1 A2 A3 W1 W2 W3
#define CMX_PIPE_WOFF(f) ((EPI == kEpiSwigluQuant ? ((f) < 2 ? (f) * 32 : 128 + ((f) - 2) * 32) : (f) * 32))
    auto read_frag = [&](auto slot_c, auto step_c, auto idx_c, v4i& lo, v4i& hi) {
        constexpr int slot = decltype(slot_c)::value, step = decltype(step_c)::value, idx = decltype(idx_c)::value;
        if constexpr (idx < 4) {
            constexpr int off = CMX_PIPE_WOFF(idx) * kSlabBytes;
            lo = lds_read_b128<off>(wb[slot][2 * step]);
            hi = lds_read_b128<off>(wb[slot][2 * step + 1]);
        } else {
            constexpr int off = (idx - 4) * 32 * kSlabBytes;
            lo = lds_read_b128<off>(ab[slot][2 * step]);
            hi = lds_read_b128<off>(ab[slot][2 * step + 1]);
        }
    };
    auto read_scale = [&](auto slot_c, auto idx_c) {
        constexpr int slot = decltype(slot_c)::value, idx = decltype(idx_c)::value;
        if constexpr (idx < 4)
            sraw[idx] = lds_read_b32<slot * kScaleSlotBytes + CMX_PIPE_WOFF(idx) * 4>(swb);
        else
            sraw[idx] = lds_read_b32<slot * kScaleSlotBytes + (idx - 4) * 32 * 4>(sab);
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // ---- prologue -------------------------------------------------------------------------------------
    {
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) issue_tile_load(0, i, 0);
        issue_scale_loads(0, 0);
        const uint32_t k1 = clamp_slab(1);
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) issue_tile_load(1, i, k1 * kSlabBytes);
        issue_scale_loads(1, k1 * 4);
        asm volatile("s_waitcnt vmcnt(18)\n\ts_barrier" ::: "memory");      // slab 0 has landed everywhere
        static_for<0, 8>([&](auto ic) {
            constexpr int idx = pipe_read_order(decltype(ic)::value);
            read_frag(I0{}, I0{}, std::integral_constant<int, idx>{}, f0lo[idx], f0hi[idx]);
        });
        static_for<0, 8>([&](auto ic) { read_scale(I0{}, ic); });
    }

    auto shift_scales = [&](auto set_c) {
        constexpr int set = decltype(set_c)::value;
        (void)scur, (void)sraw, (void)sshift;      // asm operands alone do not make a generic lambda capture
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(scur[set][i]) : "v"(sshift), "v"(sraw[i]));
    };
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    shift_scales(I0{});

    // one slab; SLOT = ring slot of slab s (compile-time so that every LDS offset is an immediate).
    // On entry fragment set 0 and the shifted scales of the slab are in registers.
    constexpr int kEarly = 7;       // tile loads of slab s+2 issued already in step 0, behind the first barrier
    auto slab_body = [&](auto slot_c, uint32_t s) {
        constexpr int slot = decltype(slot_c)::value;
        using SlotT = std::integral_constant<int, slot>;
        using OtherT = std::integral_constant<int, slot ^ 1>;
        const uint32_t k2 = clamp_slab(s + 2);
        const uint32_t koff = k2 * kSlabBytes, soff = k2 * 4;
        // ---- step 0 ----
        static_for<0, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value, fw = i / 4, fm = i % 4;
            mfma_acc<FMT, 0>(acc[fw][fm], join8(f0lo[fw], f0hi[fw]), join8(f0lo[4 + fm], f0hi[4 + fm]), scur[slot][fw], scur[slot][4 + fm]);
            if constexpr (i < 8) {
                constexpr int idx = pipe_read_order(i);
                if (!(CMX_PIPE_DBG & 4)) read_frag(SlotT{}, I1{}, std::integral_constant<int, idx>{}, f1lo[idx], f1hi[idx]);
            }
            // slot `slot` has been read for the last time: once everyone is here it can be refilled
            if constexpr (i == 16 - kEarly - 1) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if constexpr (i >= 16 - kEarly) {
                if (!(CMX_PIPE_DBG & 1)) issue_tile_load(slot, i - (16 - kEarly), koff);
            }
        });
        // own loads of slab s+1 are complete (only the kEarly loads just issued may be in flight); after the
        // barrier so are everyone's
        if (CMX_PIPE_DBG & 17) asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kEarly) : "memory");
        // ---- step 1 ----
        static_for<0, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value, fw = i / 4, fm = i % 4;
            mfma_acc<FMT, 2>(acc[fw][fm], join8(f1lo[fw], f1hi[fw]), join8(f1lo[4 + fm], f1hi[4 + fm]), scur[slot][fw], scur[slot][4 + fm]);
            if constexpr (i + kEarly < 16) {
                if (!(CMX_PIPE_DBG & 1)) issue_tile_load(slot, i + kEarly, koff);
            }
            if constexpr (i + kEarly == 16) { if (!(CMX_PIPE_DBG & 8)) issue_scale_loads(slot, soff); }
            if constexpr (i < 8) {
                constexpr int idx = pipe_read_order(i);
                if (!(CMX_PIPE_DBG & 4)) read_frag(OtherT{}, I0{}, std::integral_constant<int, idx>{}, f0lo[idx], f0hi[idx]);
            } else if constexpr (i < 12) {
                read_scale(OtherT{}, std::integral_constant<int, 2 * (i - 8)>{});
                read_scale(OtherT{}, std::integral_constant<int, 2 * (i - 8) + 1>{});
            }
            if constexpr (i == 13) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                shift_scales(OtherT{});
            }
        });
        // Keep this slab's scale registers allocated to the end of the slab: otherwise the shifts above may be
        // given the register of a scale whose last reader is an MFMA issued a few cycles earlier, and nothing
        // orders that VALU write behind the MFMA's operand fetch.
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" ::"v"(scur[slot][i]));
    };

    // The compiler does not see the MFMAs inside the asm statements, so it inserts none of the wait states
    // that separate them from its own accumulator accesses.  Passing every accumulator through an asm
    // statement that holds the wait states pins those accesses to the far side of it.
    auto fence_accumulators = [&]() {
        (void)acc;
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[0][0]), "+a"(acc[0][1]), "+a"(acc[0][2]), "+a"(acc[0][3]), "+a"(acc[1][0]), "+a"(acc[1][1]),
                       "+a"(acc[1][2]), "+a"(acc[1][3]));
        asm volatile("s_nop 15\n\ts_nop 15"
                     : "+a"(acc[2][0]), "+a"(acc[2][1]), "+a"(acc[2][2]), "+a"(acc[2][3]), "+a"(acc[3][0]), "+a"(acc[3][1]),
                       "+a"(acc[3][2]), "+a"(acc[3][3]));
    };
    fence_accumulators();       // the zero initialisation has retired before the first MFMA reads it
    for (uint32_t s = 0; s < nslab; s += 2) {      // the host only selects this kernel for an even slab count
        slab_body(I0{}, s);
        slab_body(I1{}, s + 1);
    }
    // the loads issued past the end must land before the LDS is released; the last MFMAs must have
    // written their accumulators before the epilogue reads them
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    fence_accumulators();
#undef CMX_PIPE_WOFF

    epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
}
