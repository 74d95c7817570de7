// Hand-scheduled grouped block-scaled matmul kernel for the 8-bit MX formats whose weight fragments never pass through the
// LDS (included by mx_gemm.hip after mx_gemm_pipe.h, whose helpers it shares).  Tiles of 256 weight rows x 256 or 288
// activation rows; what follows describes the 256-row form, "Tile heights" below what the taller one changes.
//
// For grouped problems with about one tile of rows per group every tile streams a weight panel of its own from HBM,
// and what bounds the two-slot kernels there is how many weight bytes a CU can keep in flight: the LDS holds two
// 64 KiB slabs, so a slab's loads have one to one and a half slab times to arrive, less than the latency of HBM under
// load.  The register file is the larger memory (512 KiB per CU against 160 KiB), and in the 4 x 1 wavefront layout the
// 64 weight rows of a wavefront are read by that wavefront alone.  So here
//   * each wavefront loads its own weight fragments straight into registers (buffer_load_dwordx4, the lane that
//     feeds a row to the MFMA fetches that row's bytes; the weights are stored pre-tiled so that such a load reads
//     whole cache lines), into a ring of FOUR slabs (128 VGPRs): the loads of slab s + 3 are issued while slab s is
//     being multiplied and have two and a half slab times to land, with up to three slabs (96 KiB per CU) in flight;
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
// The K positions are multiplied and summed in the order of the two-slot kernels (step h of a slab takes its 32-blocks
// 2h and 2h + 1), so the results are the same bits.  The lanes of half-wave lh, whose scale byte applies to the first
// (lh = 0) or second (lh = 1) block of an MFMA, need bytes lh (step 0) and 2 + lh (step 1) of the slab's dword: the dword
// is read whole, shifted right by one byte in the upper half-wave right before its first use (one VALU instruction), and
// the MFMAs select bytes 0 and 2.  The activation scale of fragment j is refreshed in place like the fragment itself.
// (Measured alternatives at 256 groups of ~256 rows, K = 7168: reading the dword at byte address lh, which the LDS
// allows, +5 % kernel time over no shift at all; the shift under a half EXEC mask +4 %; this shift +2.5 %; pairing the
// blocks (h, 2 + h), which needs no shift but sums K in another order than the other kernels and so differs from them in
// the last bit of one output in a million, +0.)
// The kernel is persistent like the two-slot grouped kernels: one workgroup per CU draws tiles from its XCD's counter,
// and the load streams run on into the next tile while the last slabs of a tile are multiplied.
#pragma once

// STREAM: bytes that this wavefront reads once and nobody else reads at all are loaded non-temporal, so that they do not
// push the activation rows, which sixteen workgroups share, out of the L2 (measured on 256 groups of ~256 rows, K = 7168,
// N = 4096: 2.14 against 2.22 ms)
template <int IMM, bool STREAM = false>
__device__ __forceinline__ v4i wreg_load_b128(uint32_t voff, v4i rsrc, uint32_t soff) {
    static_assert(IMM >= 0 && IMM < 4096, "immediate offset of a buffer load: twelve bits");
    v4i r;
    soff = __builtin_amdgcn_readfirstlane(soff);
    if constexpr (STREAM)
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4 nt" : "=v"(r) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
    else
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:%4" : "=v"(r) : "v"(voff), "s"(rsrc), "s"(soff), "n"(IMM) : "memory");
    return r;
}

// r >>= sh (sh = 8 in lanes 32..63, 0 in the others): the scale dword of a slab holds the bytes of its four 32-blocks in
// order; after this the lanes of either half-wave find their byte for step 0 (block lh) at byte 0 and that for step 1
// (block 2 + lh) at byte 2
__device__ __forceinline__ void shift_scale(uint32_t& r, uint32_t sh) {
    asm volatile("v_lshrrev_b32 %0, %1, %0" : "+v"(r) : "v"(sh));
}

// acc += W-fragment x A-fragment with scale byte BYTE (0 or 2) of both scale registers; BIT as in mfma_acc.  The
// accumulators of fragments 0..7 live in the 256 accumulation registers, which they fill; a ninth fragment's (BIT = 8, the
// 288-row tile) in ordinary vector registers, which the MFMA takes as well.
#define CMX_WREG_MFMA(ACC, SELTXT, EXTRA)                                                                       \
    asm volatile("s_bitcmp1_b32 %5, %6\n\ts_cbranch_scc0 .Lskip%=\n\t"                                          \
                 "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 " SELTXT EXTRA                        \
                 "\n.Lskip%=:"                                                                                  \
                 : ACC(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live), "n"(BIT) : "scc")
#define CMX_WREG_MFMA_SEL(ACC, EXTRA)                                                                           \
    if constexpr (BYTE == 0) { CMX_WREG_MFMA(ACC, "op_sel_hi:[0,0,0]", EXTRA); } else { CMX_WREG_MFMA(ACC, "op_sel_hi:[1,1,0]", EXTRA); }
template <int FMT, int BYTE, int BIT>
__device__ __forceinline__ void mfma_acc_b01(v16f& acc, const v8i& w, const v8i& a, uint32_t sw, uint32_t sa, uint32_t live) {
    static_assert(BYTE == 0 || BYTE == 2, "scale byte");
    static_assert(BIT >= 0 && BIT < 32, "fragment");
    live = __builtin_amdgcn_readfirstlane(live);
    if constexpr (FMT == CMX_FMT_E4M3) {
        if constexpr (BIT < 8) { CMX_WREG_MFMA_SEL("+a", ""); } else { CMX_WREG_MFMA_SEL("+v", ""); }
    } else {
        if constexpr (BIT < 8) { CMX_WREG_MFMA_SEL("+a", " cbsz:1 blgp:1"); } else { CMX_WREG_MFMA_SEL("+v", " cbsz:1 blgp:1"); }
    }
}
#undef CMX_WREG_MFMA_SEL
#undef CMX_WREG_MFMA

// Tile heights.  256 rows: eight activation fragments per wavefront, all resident in registers (each refreshed in place), the
// scales of both operands through the LDS.  288 rows: groups of up to 288 rows -- what a router that aims at 256 per expert
// mostly produces -- take one tile where the first shape needs a second one that streams the whole weight panel again for a
// few rows.  Nine fragments: their accumulators leave room for a window of three fragment buffers only (fragment j + 3 is
// read when pair j has been issued), and the LDS (four slots of 36 KiB) for the activation scales only, so the weight
// scales of a four-slab block are loaded straight into registers, 16 bytes per weight row and lane.
__host__ __device__ constexpr bool wreg_wscale_regs(int tm) { return tm != 256; }
__host__ __device__ constexpr int wreg_window(int tm) { return tm == 256 ? 8 : 3; }
__host__ __device__ constexpr int wreg_scale_rows_padded(int tm) { return ((wreg_wscale_regs(tm) ? 0 : 256) + tm + 63) / 64 * 64; }
// LDS footprint: activation ring (four slots), ring of two scale blocks (16 bytes per row), next-tile mailbox
__host__ __device__ constexpr size_t wreg_lds_bytes(int tm) { return (size_t)4 * tm * 128 + (size_t)2 * wreg_scale_rows_padded(tm) * 16 + 512; }

// LDS operations issued behind MFMA pair p of a step of kind K (0: first half of a slab, 1: second half): two fragment
// reads; in the second half preceded by the activation scale read of fragment p for the next slab, and behind pair 0 by the
// two weight scale reads as well when those go through the LDS.
__host__ __device__ constexpr int wreg_lds_ops(int kind, int p, bool wscale_regs) { return kind == 0 ? 2 : (3 + (p == 0 && !wscale_regs ? 2 : 0)); }
// lgkmcnt that guarantees fragment j of a step of kind K has landed, asked right before pair j.  With a window of `win`
// fragment buffers the reads of fragment j were the last operations behind the pair `win` pairs earlier (in this step or
// the previous one); LDS returns in order, so the count is that of the operations behind the win - 1 pairs since.  (The
// scale read of fragment j is older still.)  The counter has four bits: a smaller count only asks for older reads as well.
__host__ __device__ constexpr int wreg_frag_wait(int kind, int j, int fm, int win, bool wscale_regs) {
    int n = 0;
    for (int d = 1; d < win; ++d) {
        const int q = j - d;
        n += q >= 0 ? wreg_lds_ops(kind, q, wscale_regs) : wreg_lds_ops(1 - kind, q + fm, wscale_regs);
    }
    return n < 15 ? n : 15;
}
// loads behind pair j when `total` loads are spread over `pairs` pairs: indices [first, first + count)
__host__ __device__ constexpr int wreg_first_load(int total, int pairs, int j) { return total * j / pairs; }

// Lean 16-bit store of a 4 x 1 wavefront's accumulators (64 output columns x TM rows) in whole cache lines.  In the
// accumulator layout a lane owns, per 32 x 32 block, sixteen columns of ONE row, so a store instruction straight from the
// registers writes 32 bytes to each of 32 rows, and a line is complete only after four such instructions; the L2 has to
// hold the output and merge the pieces, at the expense of the operand lines that other workgroups are about to ask for.
// Here the 32 rows x 128 bytes that a wavefront holds for one activation fragment go through a 4 KiB staging area in the
// LDS (16-byte pieces, XOR-swizzled by row so that neither the writes nor the reads conflict) and come back with eight
// lanes on a row: a store instruction then writes eight whole lines, and it writes them non-temporal (the output is not
// read again by this kernel).  Measured on GMM2 of config 4: whole lines alone change nothing, non-temporal stores of
// the 32-byte pieces cost 16 %, the two together gain 4.4 % (1.07 against 1.12 ms).
// `stage` is the wavefront's own 8 KiB (two fragments' areas, used in turn so that a write never waits for the read before it).
template <int TW, int TM, int EPI, int FM>
__device__ __forceinline__ void lean_store_staged(const GemmParams& p, const Tile& tc, v16f (&acc)[2][FM], uint32_t ww, uint32_t lane,
                                                  uint32_t stage) {
    static_assert(epi_is_lean_store(EPI), "16-bit store epilogues only");
    const uint32_t l32 = lane & 31u, lh = lane >> 5;
    auto pack = [](float a, float b) -> uint32_t {
        if constexpr (EPI == kEpiStoreFp16) {
            typedef _Float16 v2h __attribute__((ext_vector_type(2)));
            return __builtin_bit_cast(uint32_t, (v2h){(_Float16)a, (_Float16)b});
        } else {
            return cvt_pk_bf16(a, b);
        }
    };
    // write side: row l32 of the fragment, piece (fw, qp, lh) = columns 32 fw + 16 qp + 8 lh .. + 8 of the wavefront's 64
    const uint32_t wr_row = stage + l32 * 128;
    // read side: instruction j covers rows 8 j .. 8 j + 7, lane i row 8 j + i / 8, piece i % 8
    const uint32_t rd_r = lane >> 3, rd_p = lane & 7u;
    const uint32_t col = tc.wt * TW + ww * 64 + rd_p * 8;                  // first of the lane's eight output columns
    uint16_t* const c = reinterpret_cast<uint16_t*>(p.c);
    const bool col_ok = col < p.n;                                          // n is a multiple of 8: a piece is in or out as a whole
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
        const uint32_t buf = (fm & 1) * 4096;
#pragma unroll
        for (int fw = 0; fw < 2; ++fw) {
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
                const uint32_t piece = 4 * fw + 2 * qp + lh;
                const uint32_t addr = wr_row + buf + ((piece ^ (l32 & 7u)) << 4);
                asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"((v4i){(int)s0[0], (int)s1[0], (int)s0[1], (int)s1[1]}) : "memory");
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                 // a wavefront reads only what it wrote itself: no barrier
        v4i v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = 8 * j + rd_r;
            asm volatile("ds_read_b128 %0, %1" : "=v"(v[j]) : "v"(stage + buf + r * 128 + ((rd_p ^ (r & 7u)) << 4)) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t mloc = fm * 32 + 8 * j + rd_r;
            if (mloc < tc.rows_valid && col_ok)
                __builtin_nontemporal_store(v[j], reinterpret_cast<v4i*>(c + (size_t)(tc.row0 + mloc) * p.ldc + col));
        }
    }
}

// The weights come pre-tiled (cmx_mx_pretile_weights): [group][weight tile][slab][weight wavefront][load 0..7][lane][16 bytes],
// 256 x 128 bytes per slab and tile, so that a weight load of a wavefront reads 1 KiB of consecutive bytes (eight whole cache
// lines); from row-major weights the same load takes 32 bytes from each of 32 rows, and that many more visits to the
// vector cache made the kernel a quarter slower than the two-slot ones.
template <int FMT, int EPI, int TM>
__global__ __launch_bounds__(256) void mx_gemm_wreg_kernel(const GemmParams p) {
    static_assert(FMT == CMX_FMT_E4M3 || FMT == CMX_FMT_E5M2, "8-bit element formats only");
    static_assert(EPI != kEpiStore, "persistent kernel: SwiGLU or lean 16-bit store epilogue");
    static_assert(TM == 256 || TM == 288, "tile height");
    constexpr int TW = 256, NW = 4, WW = 4, WM = 1, FW = 2;
    constexpr int FM = TM / 32;                                // activation fragments of the tile = of every wavefront
    constexpr int FMW = wreg_window(TM);                       // fragment buffers: fragment j lives in buffer j % FMW
    constexpr bool kWScaleRegs = wreg_wscale_regs(TM);
    static_assert(FM % FMW == 0 && FMW <= FM, "a fragment keeps its buffer from step to step");
    constexpr int kRing = 4;                                   // slabs in the weight register ring = slots of the activation ring
    constexpr int kSlotBytes = TM * kSlabBytes;
    constexpr int kScaleBase = kRing * kSlotBytes;
    constexpr int kScaleWRows = kWScaleRegs ? 0 : TW;          // weight rows in an LDS scale block
    constexpr int kScaleRows = kScaleWRows + TM;
    constexpr int kALoads = TM / (8 * NW);                     // LDS-DMA loads per wavefront and slab
    constexpr int kWLoads = 8;                                 // weight loads per wavefront and slab: 2 steps x 2 fragments x 2 register halves
    constexpr int kSlabLoads = kALoads + kWLoads;
    constexpr int kBlockLoads = kWScaleRegs ? 2 + FW : 2;      // loads that go out with a scale block
    static_assert(WW * WM == NW && TW % (WW * 32) == 0 && TM % (8 * NW) == 0, "tile geometry");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t ww = wave % WW, wm = wave / WW;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    // ---- tile sequence of this workgroup ---------------------------------------------------------------------------
    // Every XCD owns a contiguous run of tiles, handed out as tickets: the workgroups start with tickets 0 .. G - 1 (G =
    // workgroups per XCD) and draw further ones from the XCD's counter (or walk in strides of G when there is none).
    // Whole rounds of G tickets are one tile each.  The tiles that are left for a last, partly filled round (L of them) are
    // cut along their activation rows into S = G / L (at most 4) tickets each, so that round keeps every workgroup busy
    // for a fraction of a tile time instead of some for a whole one; a part is just a tile of TM / S rows, its sums are the
    // same bits, and the parts of a tile run side by side on one weight panel.
    const uint32_t m_tiles_all = count_m_tiles<TM>(p);
    const uint32_t total_tiles = m_tiles_all * p.w_tiles;
    uint32_t run_count;
    const uint32_t run_first = xcd_run(total_tiles, blockIdx.x % kXcds, run_count);
    const uint32_t tile_stride = gridDim.x / kXcds;                       // G
    const uint32_t full_tickets = run_count / tile_stride * tile_stride;
    const uint32_t left_tiles = run_count - full_tickets;                 // L
    constexpr uint32_t kMaxSplit = TM % 128 == 0 ? 4 : 1;                // parts of whole 32-row fragments
    const uint32_t split = left_tiles == 0 ? 1u : (tile_stride / left_tiles < kMaxSplit ? (tile_stride / left_tiles ? tile_stride / left_tiles : 1u) : kMaxSplit);
    const uint32_t split_pow2 = split >= 4 ? 4u : (split >= 2 ? 2u : 1u);
    const uint32_t run_tickets = full_tickets + left_tiles * split_pow2;
    uint32_t ticket = blockIdx.x / kXcds;
    if (ticket >= run_tickets) return;
    auto make_rsrc = [](const uint8_t* q) -> v4i {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        v4i r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));     // stride 0
        r[2] = -1;                                                           // no range limit
        r[3] = 0x00020000;
        return r;
    };
    // tile row of weight fragment f of this wavefront (SwiGLU: the gate fragment, then its up partner half a tile on)
    constexpr int kWRowsPerWave = epi_is_swiglu_quant(EPI) ? TW / 2 / WW : TW / WW;
#define CMX_WREG_WOFF(f) ((epi_is_swiglu_quant(EPI) ? ((f) < FW / 2 ? (f) * 32 : TW / 2 + ((f) - FW / 2) * 32) : (f) * 32))
    const uint32_t w_row_base = ww * kWRowsPerWave;

    // descriptors of the tile whose slabs the load streams are requesting
    v4i w_rs, a_rs, s_rs[2];
    v4i ws_rs;                                  // weight scale rows of the tile's group (weight scales in registers)
    uint32_t sgoff[2], wsgoff[FW];
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
    // Scale blocks in the LDS: the rows of both operands form one sequence (weight rows, unless those go to registers, then
    // activation rows) that is fetched in loads of 64 rows, two per wavefront: loads `wave` and `wave + 4` (where there is no
    // such load, the first again).
    constexpr int kScaleLoads = (kScaleRows + 63) / 64;
    constexpr int kScaleRowsPadded = kScaleLoads * 64;
    constexpr int kScaleSlotBytesP = kScaleRowsPadded * 16;
    const uint32_t sload[2] = {wave, wave + 4 < (uint32_t)kScaleLoads ? wave + 4 : wave};
    auto aim_scales_at = [&](const Tile& t) {
        ws_rs = make_rsrc(p.w_scale + (size_t)t.g * p.n * p.ld_ws);
        const v4i as_rs = make_rsrc(p.a_scale + (size_t)t.row0 * p.ld_as);
        if constexpr (kWScaleRegs) {
            // lane l of either half-wave: the scale row of the weight row it feeds to the MFMA as row l % 32 of fragment f
#pragma unroll
            for (int f = 0; f < FW; ++f) wsgoff[f] = mul_lo_u32(wrow_of(t, w_row_base + CMX_WREG_WOFF(f) + l32), p.ld_ws);
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const uint32_t c = 64 * sload[k] + lane;
            const bool is_w = 64 * sload[k] < (uint32_t)kScaleWRows;     // uniform: the weight rows are a multiple of 64
            const uint32_t ar = c - kScaleWRows < t.rows_valid ? c - kScaleWRows : t.rows_valid - 1;
            sgoff[k] = is_w ? wrow_of(t, c) * p.ld_ws : ar * p.ld_as;
#pragma unroll
            for (int q = 0; q < 4; ++q) s_rs[k][q] = is_w ? ws_rs[q] : as_rs[q];
        }
    };
    auto aim_tiles_at = [&](const Tile& t) {
        w_rs = make_rsrc(p.w + ((size_t)t.g * p.w_tiles + t.wt) * ((size_t)p.kbytes * TW));
        a_rs = make_rsrc(p.a + (size_t)t.row0 * p.lda);
        a_last = __builtin_amdgcn_readfirstlane(t.rows_valid - 1);
    };
    // LDS-DMA load i of this wavefront fills activation rows (4 i + wave) * 8 .. + 8; lane q -> row + q / 8, LDS chunk
    // q % 8, and fetches the global chunk that the XOR swizzle maps there (rows past the edge re-read the last one).
    // The per-lane offset is worked out in front of each load (three full-rate instructions) instead of being kept in
    // registers: row = min(first row + 32 i, last valid row), offset = row * pitch + 16 * chunk.
    const uint32_t a_row0 = wave * 8 + (lane >> 3);
    // weight load j = (step, fragment, register half) of a slab: 1 KiB at j * 1024 of this wavefront's 8 KiB of the slab
    // (one offset register per step: the immediate offset of a buffer load has twelve bits)
    const uint32_t woff[2] = {ww * 8192 + lane * 16, ww * 8192 + lane * 16 + 4096};
    const uint32_t a_chunk16 = swz(a_row0, lane & 7u) * 16;      // (row & 15) does not depend on i
    const uint32_t a_lda = __builtin_amdgcn_readfirstlane(p.lda);
    // ticket -> tile (whole, or one part of a tile of the last round); false when the part holds no rows
    auto decode_ticket = [&](uint32_t t, Tile& out, uint32_t g_from) -> bool {
        const bool whole = t < full_tickets;
        const uint32_t tile = run_first + (whole ? t : full_tickets + (t - full_tickets) / split_pow2);
        decode_tile<TM>(p, m_tiles_all, tile, out, g_from);
        if (!whole && split_pow2 > 1) {
            const uint32_t part = (t - full_tickets) % split_pow2, rpp = TM / split_pow2;
            const uint32_t skip = part * rpp;
            const uint32_t left = out.rows_valid > skip ? out.rows_valid - skip : 0u;
            out.row0 += skip;
            out.rows_valid = left < rpp ? left : rpp;
        }
        uniform_tile(out);
        return out.rows_valid != 0;
    };
    Tile tq;                                    // tile of the load streams
    while (!decode_ticket(ticket, tq, 0)) {     // (an empty part: on to this workgroup's next ticket)
        ticket += tile_stride;                  // only tickets of the last round can be empty, and those have no successors in a strided walk
        if (ticket >= run_tickets) return;
    }
    aim_scales_at(tq);
    aim_tiles_at(tq);
    Tile tc = tq;                               // tile of the MFMA stream / epilogue

    const uint32_t nslab = p.kbytes / kSlabBytes;            // a multiple of four (host check)
    const uint32_t nblk = nslab / 4;
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sdma_base[2] = {(uint32_t)__builtin_amdgcn_readfirstlane(lds0 + kScaleBase + sload[0] * 64 * 16),
                                   (uint32_t)__builtin_amdgcn_readfirstlane(lds0 + kScaleBase + sload[1] * 64 * 16)};
    auto issue_a_load = [&](auto slot_c, auto i_c, uint32_t koff) {
        constexpr int slot = decltype(slot_c)::value, i = decltype(i_c)::value;
        (void)a_row0, (void)a_chunk16, (void)a_last;
        uint32_t off;
        asm volatile("v_add_u32 %0, %1, %2\n\tv_min_u32 %0, %3, %0\n\tv_mad_u32_u24 %0, %0, %4, %5"
                     : "=&v"(off) : "n"(32 * i), "v"(a_row0), "s"(a_last), "s"(a_lda), "v"(a_chunk16));
        dma_b128(dma_base + slot * kSlotBytes + i * (NW * 1024), off, a_rs, koff);
    };
    uint32_t blocks_issued = 0;                 // running count over all tiles: ring position = count & 1
    v4i wsn[FW];                                // weight scales of the next four-slab block as they come from memory
    uint32_t wsc[FW][4];                        // ... of the current block, one register per slab, shifted for this half-wave
    auto issue_scale_block = [&](uint32_t byte_off) {
        const uint32_t pos = blocks_issued & 1u;
        ++blocks_issued;
        (void)wsn, (void)wsgoff;
        dma_b128(sdma_base[0] + pos * kScaleSlotBytesP, sgoff[0], s_rs[0], byte_off);
        dma_b128(sdma_base[1] + pos * kScaleSlotBytesP, sgoff[1], s_rs[1], byte_off);
        if constexpr (kWScaleRegs) {
#pragma unroll
            for (int f = 0; f < FW; ++f) wsn[f] = wreg_load_b128<0>(wsgoff[f], ws_rs, byte_off);
        }
    };

    // ---- fragment and scale read addresses -----------------------------------------------------------------------
    // a lane reads, for step h, the 16-byte chunks 4 h + lh (32-block 2h of the slab) and 4 h + 2 + lh (block 2h + 1) of its
    // row.  One set of four base registers serves all slots; the immediate picks the fragment.  The two bases of step 0 point
    // at the slot of slab s while step 0 of slab s is multiplied and move on to the next slot between the two steps (the last
    // reads behind the pairs of step 1 fetch the first fragments of slab s + 1); those of step 1 move on after step 1.
    const uint32_t x = (l32 & 7u) ^ ((l32 >> 3) & 1u);
    uint32_t ab[4];                             // [2 * step + half]
#pragma unroll
    for (int j = 0; j < 4; ++j) ab[j] = lds0 + (wm * 32 + l32) * kSlabBytes + ((4 * (j >> 1) + 2 * (j & 1) + lh) ^ x) * 16;
    // the bases of step `step` move on to the next slot
    auto move_read_base = [&](int step, int delta) {
        (void)ab;
#pragma unroll
        for (int j = 0; j < 2; ++j) asm volatile("v_add_u32 %0, %1, %0" : "+v"(ab[2 * step + j]) : "s"(delta));
    };
    // scale dword of the row (the lanes of half-wave lh use its bytes lh and lh + 2: see shift_scale)
    const uint32_t swb = lds0 + kScaleBase + (w_row_base + l32) * 16;
    const uint32_t sab = lds0 + kScaleBase + (kScaleWRows + wm * 32 + l32) * 16;
    const uint32_t sshift = 8 * lh;
    uint32_t blocks_read = 0;                   // running count of the scale blocks whose first slab has been read

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    v4i wlo[kRing][2][FW], whi[kRing][2][FW];           // weight ring: [slab position][step][fragment], registers 0-3 / 4-7
    v4i alo[FMW], ahi[FMW];                             // activation fragment buffers: fragment j of a step in buffer j % FMW
    uint32_t sw[2][FW];                                 // weight scales of a slab (bytes 0, 2: steps 0, 1), by slab parity (through the LDS)
    uint32_t sa[FM];                                    // activation scales, refreshed in place like the fragments

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;

    // weight load i (0..7) of a slab into ring position `pos`: step i / 4, fragment (i / 2) % 2, register half i % 2
    auto issue_w_load = [&](auto pos_c, auto i_c, uint32_t koff) {
        constexpr int pos = decltype(pos_c)::value, i = decltype(i_c)::value;
        constexpr int h = i / 4, f = (i / 2) % 2, half = i % 2;
        (void)wlo, (void)whi, (void)woff;
        v4i& dst = half ? whi[pos][h][f] : wlo[pos][h][f];
        // (with the 288-row tile nearly every group is one tile high, and its weight panel has one reader)
        dst = wreg_load_b128<(f * 2 + half) * 1024, (TM == 288)>(woff[h], w_rs, koff * TW);
    };
    // one 16-byte read of this wavefront's activation fragment j for step `step` from the slot the base registers of that step
    // point at
    auto read_a_half = [&](auto step_c, auto j_c, auto half_c) {
        constexpr int step = decltype(step_c)::value, j = decltype(j_c)::value, half = decltype(half_c)::value;
        (void)ab, (void)alo, (void)ahi;
        v4i& dst = half ? ahi[j % FMW] : alo[j % FMW];
        dst = lds_read_b128<j * WM * 32 * kSlabBytes>(ab[2 * step + half]);
    };
    // the two reads that go out behind pair j of step `step`: fragment j + FMW of that step while there is one, else fragment
    // j + FMW - FM of the step after it (whose base registers already point at its slot)
    auto read_behind = [&](auto step_c, auto j_c) {
        constexpr int step = decltype(step_c)::value, j = decltype(j_c)::value;
        constexpr int g = j + FMW;
        using StepT = std::integral_constant<int, (g < FM ? step : 1 - step)>;
        using FragT = std::integral_constant<int, (g < FM ? g : g - FM)>;
        read_a_half(StepT{}, FragT{}, I0{});
        read_a_half(StepT{}, FragT{}, I1{});
    };
    auto read_w_scale_at = [&](uint32_t swb_at, auto set_c, auto f_c) {
        constexpr int set = decltype(set_c)::value, f = decltype(f_c)::value;
        (void)sw;
        sw[set][f] = lds_read_b32<CMX_WREG_WOFF(f) * 16>(swb_at);
    };
    auto read_a_scale_at = [&](uint32_t sab_at, auto j_c) {
        constexpr int j = decltype(j_c)::value;
        (void)sa;
        sa[j] = lds_read_b32<j * WM * 32 * 16>(sab_at);
    };
    // ring position and dword of the scales of the slab that follows the one at ring position P of the MFMA stream
    auto scale_read_offset = [&](int dword) -> uint32_t {
        return __builtin_amdgcn_readfirstlane((blocks_read & 1u) * kScaleSlotBytesP + dword * 4);
    };

    // bit j: this wavefront's activation fragment j (fragment j * WM + wm of the tile) holds valid rows
    auto live_mask = [&](uint32_t rows_valid) -> uint32_t {
        const uint32_t frags = (rows_valid + 31) / 32;
        uint32_t m = 0;
#pragma unroll
        for (int j = 0; j < FM; ++j) m |= ((uint32_t)j * WM + wm < frags ? 1u : 0u) << j;
        return __builtin_amdgcn_readfirstlane(m);
    };
    uint32_t live = live_mask(tc.rows_valid);

    // ---- prologue: scale block 0, slabs 0..2 (activations before weights within a slab), fragments and scales of slab 0
    issue_scale_block(0);
    static_for<0, 3>([&](auto sc_) {
        constexpr int s = decltype(sc_)::value;
        static_for<0, kALoads>([&](auto ic) { issue_a_load(sc_, ic, s * kSlabBytes); });
        static_for<0, kWLoads>([&](auto ic) { issue_w_load(sc_, ic, s * kSlabBytes); });
    });
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kWLoads + 2 * kSlabLoads) : "memory");      // scale block 0 and the activations of slab 0 are in
    static_for<0, FMW>([&](auto fc) { read_a_half(I0{}, fc, I0{}); read_a_half(I0{}, fc, I1{}); });
    {
        const uint32_t off = scale_read_offset(0);
        if constexpr (!kWScaleRegs) static_for<0, FW>([&](auto fc) { read_w_scale_at(swb + off, I0{}, fc); });
        static_for<0, FM>([&](auto fc) { read_a_scale_at(sab + off, fc); });
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    auto fence_accumulators = [&]() {
        static_for<0, FW * FM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            (void)acc;
            if constexpr (i % FM < 8) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(acc[i / FM][i % FM]));
            else asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc[i / FM][i % FM]));
        });
    };
    fence_accumulators();

    // ---- one slab at ring position P ------------------------------------------------------------------------------
    // koff: byte offset (in the load streams' tile) of the slab that the loads issued here fetch (three ahead);
    // sblk: byte offset of the scale block issued at P = 0
    auto slab_body = [&](auto pos_c, uint32_t koff, uint32_t sblk) {
        constexpr int P = decltype(pos_c)::value;
        constexpr int kLoadSlot = (P + 3) % kRing;
        constexpr int kSet = P % 2, kNextSet = (P + 1) % 2;
        using LoadPosT = std::integral_constant<int, kLoadSlot>;
        using NextSetT = std::integral_constant<int, kNextSet>;
        (void)acc, (void)sw, (void)sa, (void)wlo, (void)whi, (void)alo, (void)ahi, (void)live, (void)sshift, (void)wsn, (void)wsc;
        // own activation loads (and scale block) of slab s + 1 have landed: younger are the weights of slab s + 1 and all of
        // slab s + 2 (plus the scale block that went out with it when that was a position-0 slab)
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kWLoads + kSlabLoads + (P == 1 ? kBlockLoads : 0)) : "memory");
        if constexpr (kWScaleRegs && P == 0) {
            // the weight scales of this turn's block arrived a turn ago: one register per slab, shifted for this half-wave
            static_for<0, FW * 4>([&](auto ic) {
                constexpr int f = decltype(ic)::value / 4, d = decltype(ic)::value % 4;
                (void)wsc, (void)wsn, (void)sshift;
                asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(wsc[f][d]) : "v"(sshift), "v"(wsn[f][d]));
            });
        }
        // scales of the next slab: dword (P + 1) % 4 of its block; a new block starts with the slab at position 0
        if constexpr (P == 3) ++blocks_read;
        const uint32_t sc_off = scale_read_offset((P + 1) % 4);
        const uint32_t swb_at = swb + sc_off, sab_at = sab + sc_off;
        // ---- step 0 ----
        static_for<0, FM>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(wreg_frag_wait(0, j, FM, FMW, kWScaleRegs)) : "memory");
            // the scales of this slab were read from the LDS as whole dwords (behind the pairs of the previous step): first use here
            if constexpr (j == 0 && !kWScaleRegs) {
                shift_scale(sw[kSet][0], sshift);
                shift_scale(sw[kSet][1], sshift);
            }
            shift_scale(sa[j], sshift);
            const v8i a = join8(alo[j % FMW], ahi[j % FMW]);
            mfma_acc_b01<FMT, 0, j>(acc[0][j], join8(wlo[P][0][0], whi[P][0][0]), a, kWScaleRegs ? wsc[0][P] : sw[kSet][0], sa[j], live);
            mfma_acc_b01<FMT, 0, j>(acc[1][j], join8(wlo[P][0][1], whi[P][0][1]), a, kWScaleRegs ? wsc[1][P] : sw[kSet][1], sa[j], live);
            read_behind(I0{}, jc);
            if constexpr (P == 0 && j == 0) issue_scale_block(sblk);
            static_for<wreg_first_load(kALoads, FM, j), wreg_first_load(kALoads, FM, j + 1)>([&](auto ic) { issue_a_load(LoadPosT{}, ic, koff); });
        });
        move_read_base(0, P == 3 ? -3 * kSlotBytes : kSlotBytes);
        // ---- step 1 ----
        static_for<0, FM>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(wreg_frag_wait(1, j, FM, FMW, kWScaleRegs)) : "memory");
            const v8i a = join8(alo[j % FMW], ahi[j % FMW]);
            mfma_acc_b01<FMT, 2, j>(acc[0][j], join8(wlo[P][1][0], whi[P][1][0]), a, kWScaleRegs ? wsc[0][P] : sw[kSet][0], sa[j], live);
            mfma_acc_b01<FMT, 2, j>(acc[1][j], join8(wlo[P][1][1], whi[P][1][1]), a, kWScaleRegs ? wsc[1][P] : sw[kSet][1], sa[j], live);
            if constexpr (j == 0 && !kWScaleRegs) {
                read_w_scale_at(swb_at, NextSetT{}, I0{});
                read_w_scale_at(swb_at, NextSetT{}, I1{});
            }
            read_a_scale_at(sab_at, jc);
            read_behind(I1{}, jc);
            static_for<wreg_first_load(kWLoads, FM, j), wreg_first_load(kWLoads, FM, j + 1)>([&](auto ic) { issue_w_load(LoadPosT{}, ic, koff); });
        });
        move_read_base(1, P == 3 ? -3 * kSlotBytes : kSlotBytes);
    };

    // ---- persistent loop: four slabs per turn, tiles change between turns ------------------------------------------
    uint32_t sm = 0;                 // first slab of the turn within the MFMA stream's tile
    bool next_ok = false;
    Tile tn = tq;
    for (;;) {
        const bool last_turn = sm + 4 == nslab;
        uint32_t k1, k2, k3, sblk;
        const uint32_t k0 = (sm + 3) * kSlabBytes;            // position 0 always requests a slab of the current tile
        if (last_turn) {
            // the load streams are about to run out of this tile: the next one (positions 1..3 and the scale block)
            next_ok = false;
            for (;;) {
                if (p.tile_ctr != nullptr) {
                    uint32_t* const mailbox = reinterpret_cast<uint32_t*>(smem + kScaleBase + 2 * kScaleSlotBytesP);
                    if (tid == 0) *mailbox = atomicAdd(reinterpret_cast<unsigned int*>(p.tile_ctr) + blockIdx.x % kXcds, 1u);
                    __syncthreads();
                    ticket = tile_stride + __builtin_amdgcn_readfirstlane(*mailbox);
                    __syncthreads();                                     // everyone has read the mailbox before it is written again
                } else {
                    ticket += tile_stride;
                }
                if (ticket >= run_tickets) break;
                if (decode_ticket(ticket, tn, tq.g)) {                   // tickets only grow, and with them the groups
                    next_ok = true;
                    break;
                }
            }
            if (next_ok) {
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
            if constexpr (epi_is_lean_store(EPI)) {
                // the slot of the slab just multiplied (ring position 3) is free once every wavefront has read its last
                // fragments, and stays free until the barrier at the start of the next slab: 8 KiB of it per wavefront
                __builtin_amdgcn_s_barrier();
                lean_store_staged<TW, TM, EPI, FM>(p, tc, acc, ww, lane, lds0 + 3 * kSlotBytes + wave * 8192);
            } else {
                epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
            }
            if (!next_ok) break;
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
            // first fragments of the new tile again (slot 0 has landed and is visible, and the base registers point at it;
            // the activation scales of its slab 0 are already in their registers, the weight scales in theirs or on their way)
            static_for<0, FMW>([&](auto fc) { read_a_half(I0{}, fc, I0{}); read_a_half(I0{}, fc, I1{}); });
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // the re-requested slabs land before the LDS is released
#undef CMX_WREG_WOFF
}
