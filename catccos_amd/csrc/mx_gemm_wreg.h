// Hand-scheduled 256 x 256 block-scaled matmul kernel for the 8-bit MX formats whose weight fragments never pass
// through the LDS (included by mx_gemm.hip after mx_gemm_pipe.h, whose helpers it shares).
//
// For grouped problems with about one tile of rows per group every tile streams a weight panel of its own from HBM,
// and what bounds the two-slot kernels there is how many weight bytes a CU can keep in flight: the LDS holds two
// 64 KiB slabs, so a slab's loads have one to one and a half slab times to arrive, less than the latency of HBM under
// load.  The register file is the larger memory (512 KiB per CU against 160 KiB), and in the 4 x 1 wavefront layout the
// 64 weight rows of a wavefront are read by that wavefront alone.  So here
//   * each wavefront loads its own weight fragments straight into registers (buffer_load_dwordx4, the lane that
//     feeds a row to the MFMA fetches that row's bytes), into a ring of FOUR slabs (128 VGPRs): the loads of slab
//     s + 3 are issued while slab s is being multiplied and have two and a half slab times to land, with up to three
//     slabs (96 KiB per CU) in flight;
//   * only the activation rows, which all four wavefronts read, go through the LDS (LDS-DMA into a ring of four
//     32 KiB slots, three slabs ahead as well), together with the scale blocks of both operands;
//   * the eight activation fragments of a step are refreshed in place: fragment j of the next step is read as soon
//     as the two MFMAs that use fragment j of this step have been issued (the data comes back a hundred clocks later,
//     long after those MFMAs have fetched their operands), so one set of fragment registers (64) is enough.
// One barrier per slab: at the start of slab s every wavefront has waited for its own activation loads of slab
// s + 1 (they are two slabs old) and has finished slab s - 1, so the barrier both publishes slab s + 1 and frees the
// slot of slab s - 1 for the loads of slab s + 3.  Vector memory returns in order: within a slab the activation loads
// are issued before the weight loads, so that the wait for the activations of slab s + 1 leaves the younger weight
// loads (slabs s + 1 and s + 2) in flight.
//
// Per slab s (ring position P = s mod 4, both rings), per wavefront:
//   start:   s_waitcnt vmcnt(24 or 26) + barrier
//   step 0:  8 pairs of MFMAs (activation fragment j against the two weight fragments); behind pair j the two reads
//            of fragment j for step 1 and LDS-DMA load j of the activation rows of slab s + 3 (at P = 0 also the next
//            scale block, two loads)
//   step 1:  8 pairs; behind pair j the scale read and the two reads of fragment j of slab s + 1 (pair 0: also the two
//            weight scales) and weight load j of slab s + 3
// Scales need no byte shift here: a step multiplies the slab's 32-blocks (h, 2 + h) instead of (2h, 2h + 1) -- any
// assignment of K positions to steps serves, as long as both operands use the same -- so the lanes of half-wave lh,
// whose scale byte applies to the first (lh = 0) or second (lh = 1) block of an MFMA, find their bytes for step 0 and
// step 1 side by side at byte 2 lh of the slab's dword: one ds_read_u16 per fragment, byte select 0 or 1 in the MFMA,
// and the activation scale of fragment j is refreshed in place like the fragment itself.
// The kernel is persistent like the two-slot grouped kernels: one workgroup per CU draws tiles from its XCD's counter,
// and the load streams run on into the next tile while the last slabs of a tile are multiplied.
#pragma once

template <int IMM>
__device__ __forceinline__ v4i wreg_load_b128(uint32_t voff, v4i rsrc, uint32_t soff) {
    v4i r;
    soff = __builtin_amdgcn_readfirstlane(soff);
#if defined(CMX_WREG_WPOL) && CMX_WREG_WPOL == 1
#define CMX_WREG_WPOLICY " nt"
#elif defined(CMX_WREG_WPOL) && CMX_WREG_WPOL == 2
#define CMX_WREG_WPOLICY " sc1 nt"
#elif defined(CMX_WREG_WPOL) && CMX_WREG_WPOL == 3
#define CMX_WREG_WPOLICY " sc0 sc1"
#else
#define CMX_WREG_WPOLICY ""
#endif
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" CMX_WREG_WPOLICY : "=v"(r) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
    return r;
}

template <int OFF>
__device__ __forceinline__ uint32_t lds_read_u16(uint32_t addr) {
    uint32_t r;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}

// acc += W-fragment x A-fragment with scale byte BYTE (0 or 1) of both scale registers; BIT as in mfma_acc
#define CMX_WREG_MFMA(SELTXT, EXTRA)                                                                            \
    if constexpr (BIT < 0)                                                                                      \
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 " SELTXT EXTRA                    \
                     : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));                                           \
    else                                                                                                        \
        asm volatile("s_bitcmp1_b32 %5, %6\n\ts_cbranch_scc0 .Lskip%=\n\t"                                      \
                     "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 " SELTXT EXTRA                    \
                     "\n.Lskip%=:"                                                                              \
                     : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live), "n"(BIT < 0 ? 0 : BIT) : "scc")
template <int FMT, int BYTE, int BIT>
__device__ __forceinline__ void mfma_acc_b01(v16f& acc, const v8i& w, const v8i& a, uint32_t sw, uint32_t sa, uint32_t live) {
    static_assert(BYTE == 0 || BYTE == 1, "scale byte");
    live = __builtin_amdgcn_readfirstlane(live);
#ifdef CMX_WREG_NO_MFMA
    asm volatile("" : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live));
    return;
#endif
    if constexpr (FMT == CMX_FMT_E4M3) {
        if constexpr (BYTE == 0) { CMX_WREG_MFMA("op_sel_hi:[0,0,0]", ""); } else { CMX_WREG_MFMA("op_sel:[1,1,0] op_sel_hi:[0,0,0]", ""); }
    } else {
        if constexpr (BYTE == 0) { CMX_WREG_MFMA("op_sel_hi:[0,0,0]", " cbsz:1 blgp:1"); } else { CMX_WREG_MFMA("op_sel:[1,1,0] op_sel_hi:[0,0,0]", " cbsz:1 blgp:1"); }
    }
}
#undef CMX_WREG_MFMA

// LDS operations issued behind MFMA pair p of a step of kind K (0: first half of a slab, 1: second half): two fragment
// reads; in the second half preceded by the scale read of that fragment for the next slab, and behind pair 0 by the two
// weight scale reads as well.
__host__ __device__ constexpr int wreg_lds_ops(int kind, int p) { return kind == 0 ? 2 : (3 + (p == 0 ? 2 : 0)); }
// lgkmcnt that guarantees fragments j and j + 1 of a step of kind K (and with them the scales read before them) have
// landed, asked right before pair j (j even): LDS returns in order, so it is the number of operations issued after the
// reads of fragment j + 1 -- the rest of the previous step (kind 1 - K) and pairs 0..j-1 of this one.
__host__ __device__ constexpr int wreg_frag_wait(int kind, int j) {
    int n = 0;
    for (int p = j + 2; p < 8; ++p) n += wreg_lds_ops(1 - kind, p);
    for (int p = 0; p < j; ++p) n += wreg_lds_ops(kind, p);
    return n < 15 ? n : 15;                    // the counter has four bits: a smaller count only asks for older reads as well
}

// PRE: the weights come pre-tiled (cmx_mx_pretile_weights): [group][weight tile][slab][wavefront][load 0..7][lane][16 bytes],
// 32 KiB per slab and tile, so that a weight load of a wavefront reads 1 KiB of consecutive bytes (eight whole cache lines)
// instead of 32 bytes from each of 32 rows.
template <int FMT, int EPI, bool PRE>
__global__ __launch_bounds__(256) void mx_gemm_wreg_kernel(const GemmParams p) {
    static_assert(FMT == CMX_FMT_E4M3 || FMT == CMX_FMT_E5M2, "8-bit element formats only");
    static_assert(EPI != kEpiStore, "persistent kernel: SwiGLU or lean 16-bit store epilogue");
    constexpr int TW = 256, TM = 256, NW = 4, WW = 4, WM = 1, FW = 2, FM = 8, NF = FW + FM;
    constexpr int kRing = 4;                                   // slabs in the weight register ring = slots of the activation ring
    constexpr int kSlotBytes = TM * kSlabBytes;                // 32 KiB
    constexpr int kScaleBase = kRing * kSlotBytes;
    constexpr int kScaleRows = TW + TM;
    constexpr int kScaleSlotBytes = kScaleRows * 16;           // one block: 16 bytes (the scales of four slabs) per row
    constexpr int kScaleRingBytes = 2 * kScaleSlotBytes;
    constexpr int kALoads = TM / (8 * NW);                     // LDS-DMA loads per wavefront and slab (8)
    static_assert(kALoads == 8 && FM == 8, "one activation load and one weight load behind every MFMA pair");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t ww = wave;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    // ---- tile sequence of this workgroup (as in the two-slot persistent kernels) -----------------------------------
    const uint32_t m_tiles_all = count_m_tiles<TM>(p);
    const uint32_t total_tiles = m_tiles_all * p.w_tiles;
    uint32_t run_count;
    const uint32_t run_first = xcd_run(total_tiles, blockIdx.x % kXcds, run_count);
    const uint32_t run_end = run_first + run_count;
    const uint32_t tile_stride = gridDim.x / kXcds;
    uint32_t tile_id = run_first + blockIdx.x / kXcds;
    if (tile_id >= run_end) return;

    auto make_rsrc = [](const uint8_t* q) -> v4i {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        v4i r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));     // stride 0
        r[2] = -1;                                                           // no range limit
        r[3] = 0x00020000;
        return r;
    };
    // tile row of weight fragment f of this wavefront (SwiGLU: the gate fragment, then its up partner 128 rows on)
    constexpr int kWRowsPerWave = epi_is_swiglu_quant(EPI) ? TW / 2 / WW : TW / WW;
#define CMX_WREG_WOFF(f) ((epi_is_swiglu_quant(EPI) ? ((f) < FW / 2 ? (f) * 32 : TW / 2 + ((f) - FW / 2) * 32) : (f) * 32))
    const uint32_t w_row_base = ww * kWRowsPerWave;

    // descriptors of the tile whose slabs the load streams are requesting
    v4i w_rs, a_rs, ws_rs, as_rs;
    uint32_t woff[FW], sgoff_w, sgoff_a;
    uint32_t a_last = 0;                        // last valid activation row of that tile
    auto wrow_of = [&](const Tile& t, uint32_t r) -> uint32_t {
        uint32_t gr;
        if (epi_is_swiglu_quant(EPI)) {
            const uint32_t half = p.n >> 1;
            uint32_t rr = r < TW / 2 ? t.wt * (TW / 2) + r : t.wt * (TW / 2) + (r - TW / 2);
            rr = rr < half ? rr : half - 1;
            gr = r < TW / 2 ? rr : half + rr;
        } else {
            gr = t.wt * TW + r;
            gr = gr < p.n ? gr : p.n - 1;
        }
        return gr;
    };
    auto uniform_tile = [](Tile& t) {
        t.g = __builtin_amdgcn_readfirstlane(t.g); t.wt = __builtin_amdgcn_readfirstlane(t.wt);
        t.mt = __builtin_amdgcn_readfirstlane(t.mt); t.row0 = __builtin_amdgcn_readfirstlane(t.row0);
        t.rows_valid = __builtin_amdgcn_readfirstlane(t.rows_valid);
    };
    // scale blocks: this wavefront fetches those of weight rows 64 * wave .. and of activation rows 64 * wave ..
    auto aim_scales_at = [&](const Tile& t) {
        ws_rs = make_rsrc(p.w_scale + (size_t)t.g * p.n * p.ld_ws);
        as_rs = make_rsrc(p.a_scale + (size_t)t.row0 * p.ld_as);
        const uint32_t ar = 64 * wave + lane;
        sgoff_w = wrow_of(t, 64 * wave + lane) * p.ld_ws;
        sgoff_a = (ar < t.rows_valid ? ar : t.rows_valid - 1) * p.ld_as;
    };
    auto aim_tiles_at = [&](const Tile& t) {
#ifdef CMX_WREG_SAME_W
        if constexpr (PRE) w_rs = make_rsrc(p.w);
#else
        if constexpr (PRE) w_rs = make_rsrc(p.w + ((size_t)t.g * p.w_tiles + t.wt) * ((size_t)p.kbytes * TW));
#endif
        else w_rs = make_rsrc(p.w + (size_t)t.g * p.n * p.ldw);
#ifdef CMX_WREG_SAME_A
        a_rs = make_rsrc(p.a);
#else
        a_rs = make_rsrc(p.a + (size_t)t.row0 * p.lda);
#endif
        // weight fragment f, lane l: row l % 32 of the fragment, bytes 16 * (l / 32) + {0, 32, 64, 96} of the slab
#pragma unroll
        for (int f = 0; f < FW; ++f) {
            if constexpr (PRE) woff[f] = wave * 8192 + lane * 16 + f * 4096;         // pre-tiled: index = step, not fragment
            else woff[f] = mul_lo_u32(wrow_of(t, w_row_base + CMX_WREG_WOFF(f) + l32), p.ldw) + lh * 16;
        }
        a_last = __builtin_amdgcn_readfirstlane(t.rows_valid - 1);
    };
    // LDS-DMA load i of this wavefront fills activation rows (4 i + wave) * 8 .. + 8; lane q -> row + q / 8, LDS chunk
    // q % 8, and fetches the global chunk that the XOR swizzle maps there (rows past the edge re-read the last one).
    // The per-lane offset is worked out in front of each load (three full-rate instructions) instead of being kept in
    // eight registers: row = min(first row + 32 i, last valid row), offset = row * pitch + 16 * chunk.
    const uint32_t a_row0 = wave * 8 + (lane >> 3);
    const uint32_t a_chunk16 = swz(a_row0, lane & 7u) * 16;      // (row & 15) does not depend on i
    const uint32_t a_lda = __builtin_amdgcn_readfirstlane(p.lda);
    Tile tq;                                    // tile of the load streams
    decode_tile<TM>(p, m_tiles_all, tile_id, tq, 0);
    uniform_tile(tq);
    aim_scales_at(tq);
    aim_tiles_at(tq);
    Tile tc = tq;                               // tile of the MFMA stream / epilogue

    const uint32_t nslab = p.kbytes / kSlabBytes;            // a multiple of four (host check)
    const uint32_t nblk = nslab / 4;
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sdma_base_w = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + wave * 64 * 16);
    const uint32_t sdma_base_a = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + (TW + wave * 64) * 16);
    auto issue_a_load = [&](auto slot_c, auto i_c, uint32_t koff) {
        constexpr int slot = decltype(slot_c)::value, i = decltype(i_c)::value;
        (void)a_row0, (void)a_chunk16, (void)a_last;
        uint32_t off;
        asm volatile("v_add_u32 %0, %1, %2\n\tv_min_u32 %0, %3, %0\n\tv_mad_u32_u24 %0, %0, %4, %5"
                     : "=&v"(off) : "n"(32 * i), "v"(a_row0), "s"(a_last), "s"(a_lda), "v"(a_chunk16));
        dma_b128(dma_base + slot * kSlotBytes + i * (NW * 1024), off, a_rs, koff);
    };
    uint32_t blocks_issued = 0;                 // running count over all tiles: ring position = count & 1
    auto issue_scale_block = [&](uint32_t byte_off) {
        const uint32_t pos = blocks_issued & 1u;
        ++blocks_issued;
        dma_b128(sdma_base_w + pos * kScaleSlotBytes, sgoff_w, ws_rs, byte_off);
        dma_b128(sdma_base_a + pos * kScaleSlotBytes, sgoff_a, as_rs, byte_off);
    };

    // ---- fragment and scale read addresses -----------------------------------------------------------------------
    // a lane reads, for step h, the 16-byte chunks 2 h + lh (32-block h of the slab) and 4 + 2 h + lh (block 2 + h).  An
    // LDS offset is a 16-bit immediate, so slots 0-1 and 2-3 need different base registers: one set of four, moved by
    // 64 KiB twice per turn of four slabs
    const uint32_t x = (l32 & 7u) ^ ((l32 >> 3) & 1u);
    uint32_t ab[4];                             // [2 * step + half]
#pragma unroll
    for (int j = 0; j < 4; ++j) ab[j] = lds0 + l32 * kSlabBytes + ((2 * (j >> 1) + lh + 4 * (j & 1)) ^ x) * 16;
    auto move_read_base = [&](int delta) {
        (void)ab;
#pragma unroll
        for (int j = 0; j < 4; ++j) asm volatile("v_add_u32 %0, %1, %0" : "+v"(ab[j]) : "s"(delta));
    };
    // scale bytes of this half-wave for the two steps of a slab: bytes 2 lh, 2 lh + 1 of the row's dword
    const uint32_t swb = lds0 + kScaleBase + (w_row_base + l32) * 16 + 2 * lh;
    const uint32_t sab = lds0 + kScaleBase + (TW + l32) * 16 + 2 * lh;
    uint32_t blocks_read = 0;                   // running count of the scale blocks whose first slab has been read

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    v4i wlo[kRing][2][FW], whi[kRing][2][FW];           // weight ring: [slab position][step][fragment], registers 0-3 / 4-7
    v4i alo[FM], ahi[FM];                               // the activation fragments of the step being multiplied (refreshed in place)
    uint32_t sw[2][FW];                                 // weight scales of a slab (bytes 0, 1: steps 0, 1), by slab parity
    uint32_t sa[FM];                                    // activation scales, refreshed in place like the fragments

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // weight load i (0..7) of a slab into ring position `pos`: step i / 4, fragment (i / 2) % 2, register half i % 2
    auto issue_w_load = [&](auto pos_c, auto i_c, uint32_t koff) {
        constexpr int pos = decltype(pos_c)::value, i = decltype(i_c)::value;
        constexpr int h = i / 4, f = (i / 2) % 2, half = i % 2;
        (void)wlo, (void)whi, (void)woff;
        v4i& dst = half ? whi[pos][h][f] : wlo[pos][h][f];
        if constexpr (PRE) dst = wreg_load_b128<(f * 2 + half) * 1024>(woff[h], w_rs, koff * TW);
        else dst = wreg_load_b128<h * 32 + half * 64>(woff[f], w_rs, koff);
    };
    // one 16-byte read of activation fragment fm for step `step` of the slab in slot `slot`
    auto read_a_half = [&](auto slot_c, auto step_c, auto fm_c, auto half_c) {
        constexpr int slot = decltype(slot_c)::value, step = decltype(step_c)::value, fm = decltype(fm_c)::value, half = decltype(half_c)::value;
        (void)ab, (void)alo, (void)ahi;
        v4i& dst = half ? ahi[fm] : alo[fm];
        dst = lds_read_b128<(slot % 2) * kSlotBytes + fm * 32 * kSlabBytes>(ab[2 * step + half]);
    };
    auto read_w_scale_at = [&](uint32_t swb_at, auto set_c, auto f_c) {
        constexpr int set = decltype(set_c)::value, f = decltype(f_c)::value;
        (void)sw;
        sw[set][f] = lds_read_u16<CMX_WREG_WOFF(f) * 16>(swb_at);
    };
    auto read_a_scale_at = [&](uint32_t sab_at, auto fm_c) {
        constexpr int fm = decltype(fm_c)::value;
        (void)sa;
        sa[fm] = lds_read_u16<fm * 32 * 16>(sab_at);
    };
    // ring position and dword of the scales of the slab that follows the one at ring position P of the MFMA stream
    auto scale_read_offset = [&](int dword) -> uint32_t {
        return __builtin_amdgcn_readfirstlane((blocks_read & 1u) * kScaleSlotBytes + dword * 4);
    };

    auto live_mask = [](uint32_t rows_valid) -> uint32_t { return __builtin_amdgcn_readfirstlane((1u << ((rows_valid + 31) / 32)) - 1u); };
    uint32_t live = live_mask(tc.rows_valid);      // bit fm: activation block fm of the tile holds valid rows

    // ---- prologue: scale block 0, slabs 0..2 (activations before weights within a slab), fragments and scales of slab 0
    issue_scale_block(0);
    static_for<0, 3>([&](auto sc_) {
        constexpr int s = decltype(sc_)::value;
        static_for<0, kALoads>([&](auto ic) { issue_a_load(sc_, ic, s * kSlabBytes); });
        static_for<0, 8>([&](auto ic) { issue_w_load(sc_, ic, s * kSlabBytes); });
    });
    asm volatile("s_waitcnt vmcnt(40)\n\ts_barrier" ::: "memory");          // scale block 0 and the activations of slab 0 are in
    static_for<0, FM>([&](auto fc) { read_a_half(I0{}, I0{}, fc, I0{}); read_a_half(I0{}, I0{}, fc, I1{}); });
    {
        const uint32_t off = scale_read_offset(0);
        static_for<0, FW>([&](auto fc) { read_w_scale_at(swb + off, I0{}, fc); });
        static_for<0, FM>([&](auto fc) { read_a_scale_at(sab + off, fc); });
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    auto fence_accumulators = [&]() {
        v16f* const a = &acc[0][0];
        asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]), "+a"(a[4]), "+a"(a[5]), "+a"(a[6]), "+a"(a[7]));
        asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[8]), "+a"(a[9]), "+a"(a[10]), "+a"(a[11]), "+a"(a[12]), "+a"(a[13]), "+a"(a[14]), "+a"(a[15]));
    };
    fence_accumulators();

    // ---- one slab at ring position P ------------------------------------------------------------------------------
    // koff: byte offset (in the load streams' tile) of the slab that the loads issued here fetch (three ahead);
    // sblk: byte offset of the scale block issued at P = 0
    auto slab_body = [&](auto pos_c, uint32_t koff, uint32_t sblk) {
        constexpr int P = decltype(pos_c)::value;
        constexpr int kNextSlot = (P + 1) % kRing, kLoadSlot = (P + 3) % kRing;
        constexpr int kSet = P % 2, kNextSet = (P + 1) % 2;
        using PosT = std::integral_constant<int, P>;
        using NextSlotT = std::integral_constant<int, kNextSlot>;
        using LoadPosT = std::integral_constant<int, kLoadSlot>;
        using NextSetT = std::integral_constant<int, kNextSet>;
        (void)acc, (void)sw, (void)sa, (void)wlo, (void)whi, (void)alo, (void)ahi, (void)live;
        // own activation loads (and scale block) of slab s + 1 have landed: younger are the weights of slab s + 1 and all of
        // slab s + 2 (plus the scale block that went out with it when that was a position-0 slab)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(24 + (P == 1 ? 2 : 0)) : "memory");
        // scales of the next slab: dword (P + 1) % 4 of its block; a new block starts with the slab at position 0
        if constexpr (P == 3) ++blocks_read;
        const uint32_t sc_off = scale_read_offset((P + 1) % 4);
        const uint32_t swb_at = swb + sc_off, sab_at = sab + sc_off;
        // ---- step 0 ----
        static_for<0, FM>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if constexpr (j % 2 == 0) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(wreg_frag_wait(0, j)) : "memory");
            const v8i a = join8(alo[j], ahi[j]);
            mfma_acc_b01<FMT, 0, j>(acc[0][j], join8(wlo[P][0][0], whi[P][0][0]), a, sw[kSet][0], sa[j], live);
            mfma_acc_b01<FMT, 0, j>(acc[1][j], join8(wlo[P][0][1], whi[P][0][1]), a, sw[kSet][1], sa[j], live);
            read_a_half(PosT{}, I1{}, jc, I0{});
            read_a_half(PosT{}, I1{}, jc, I1{});
            if constexpr (P == 0 && j == 0) issue_scale_block(sblk);
            issue_a_load(LoadPosT{}, jc, koff);
        });
        // the fragment reads of step 1 go to the next slab's slot: slots 0-1 and 2-3 have different base addresses
        if constexpr (P == 1) move_read_base(2 * kSlotBytes);
        if constexpr (P == 3) move_read_base(-2 * kSlotBytes);
        // ---- step 1 ----
        static_for<0, FM>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            if constexpr (j % 2 == 0) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(wreg_frag_wait(1, j)) : "memory");
            const v8i a = join8(alo[j], ahi[j]);
            mfma_acc_b01<FMT, 1, j>(acc[0][j], join8(wlo[P][1][0], whi[P][1][0]), a, sw[kSet][0], sa[j], live);
            mfma_acc_b01<FMT, 1, j>(acc[1][j], join8(wlo[P][1][1], whi[P][1][1]), a, sw[kSet][1], sa[j], live);
            if constexpr (j == 0) {
                read_w_scale_at(swb_at, NextSetT{}, I0{});
                read_w_scale_at(swb_at, NextSetT{}, I1{});
            }
            read_a_scale_at(sab_at, jc);
            read_a_half(NextSlotT{}, I0{}, jc, I0{});
            read_a_half(NextSlotT{}, I0{}, jc, I1{});
            issue_w_load(LoadPosT{}, jc, koff);
        });
    };

    // ---- persistent loop: four slabs per turn, tiles change between turns ------------------------------------------
    uint32_t sm = 0;                 // first slab of the turn within the MFMA stream's tile
    bool next_ok = false;
    uint32_t next_id = tile_id;
    Tile tn = tq;
    for (;;) {
        const bool last_turn = sm + 4 == nslab;
        uint32_t k1, k2, k3, sblk;
        const uint32_t k0 = (sm + 3) * kSlabBytes;            // position 0 always requests a slab of the current tile
        if (last_turn) {
            // the load streams are about to run out of this tile: the next one (positions 1..3 and the scale block)
            if (p.tile_ctr != nullptr) {
                uint32_t* const mailbox = reinterpret_cast<uint32_t*>(smem + kScaleBase + kScaleRingBytes);
                if (tid == 0) *mailbox = atomicAdd(reinterpret_cast<unsigned int*>(p.tile_ctr) + blockIdx.x % kXcds, 1u);
                __syncthreads();
                next_id = run_first + tile_stride + __builtin_amdgcn_readfirstlane(*mailbox);
            } else {
                next_id = tile_id + tile_stride;
            }
            next_ok = next_id < run_end;
            if (next_ok) {
                decode_tile<TM>(p, m_tiles_all, next_id, tn, tq.g);      // tile ids only grow
                uniform_tile(tn);
                aim_scales_at(tn);
                sblk = 0;
                k1 = 0; k2 = kSlabBytes; k3 = 2 * kSlabBytes;
            } else {
                sblk = (nblk - 1) * 16;                                  // nothing new to request: harmless re-requests
                k1 = k2 = k3 = (nslab - 1) * kSlabBytes;
            }
        } else {
            sblk = (sm / 4 + 1) * 16;
            k1 = (sm + 4) * kSlabBytes; k2 = (sm + 5) * kSlabBytes; k3 = (sm + 6) * kSlabBytes;
        }
        slab_body(std::integral_constant<int, 0>{}, k0, sblk);
        if (last_turn && next_ok) {
            aim_tiles_at(tn);
            tq = tn;
        }
        slab_body(std::integral_constant<int, 1>{}, k1, 0);
        slab_body(std::integral_constant<int, 2>{}, k2, 0);
        slab_body(std::integral_constant<int, 3>{}, k3, 0);
        sm += 4;
        if (sm == nslab) {
            // the reads issued behind the last MFMAs target fragment registers that are dead on this path
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            fence_accumulators();
            epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, 0, lane);
            if (!next_ok) break;
            tile_id = next_id;
            tc = tq;
            live = live_mask(tc.rows_valid);
            next_ok = false;
            sm = 0;
#pragma unroll
            for (int i = 0; i < FW; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
            fence_accumulators();
            // first fragments of the new tile again (slot 0 has landed and is visible; the scales of its slab 0 are
            // already in their registers)
            static_for<0, FM>([&](auto fc) { read_a_half(I0{}, I0{}, fc, I0{}); read_a_half(I0{}, I0{}, fc, I1{}); });
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // the re-requested slabs land before the LDS is released
#undef CMX_WREG_WOFF
}
