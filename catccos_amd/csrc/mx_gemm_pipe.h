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
// One slab = 128 bytes of K = two MFMA steps.  Per slab s (ring slot s%2) and wavefront:
//   step 0: 16 MFMAs on fragment set 0.  Behind the first 8 go the 16 reads of fragment set 1 (second half
//           of the slab); after MFMA 8 those reads have landed, and a first barrier says that everybody is
//           done with the slot, so the loads of slab s+2 into it start right away (7 behind the remaining
//           MFMAs).  The step ends with the wait for the own loads of slab s+1 (the 7 just issued may stay in
//           flight) and a second barrier that makes slab s+1 visible to all.
//   step 1: 16 MFMAs on fragment set 1.  Behind them the other 9+2 loads of slab s+2, the 16 reads of
//           fragment set 0 from slab s+1, its 8 scale dwords and their per-half-wave byte shift.
// A load is thus in flight for 23 to 38 MFMA times before anyone waits for it.  (The grouped two-slot kernels read the
// second half's weight fragments first, free the weight rows of the slot with a barrier after MFMA 4 (2 x 2) or 2 (4 x 1)
// and send all eight weight loads of slab s+2 behind the following MFMAs; the persistent 2 x 2 kernels also issue two L2
// prefetch loads per slab in step 1: see kWFirst and CMX_PIPE_PREFETCH below.)
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

// 32-bit product in one register (the compiler's own choice for "a * b + c" is the 64-bit multiply-add, whose
// result occupies a register pair for as long as the offset lives)
__device__ __forceinline__ uint32_t mul_lo_u32(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_mul_lo_u32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
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
// lds_dst and soff are wavefront-uniform; readfirstlane makes that visible to the register allocator, which
// otherwise may hand a vector register to an "s" operand.
__device__ __forceinline__ void dma_b128(uint32_t lds_dst, uint32_t voff, v4i rsrc, uint32_t soff) {
    lds_dst = __builtin_amdgcn_readfirstlane(lds_dst);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}
__device__ __forceinline__ void dma_b32(uint32_t lds_dst, uint32_t voff, v4i rsrc, uint32_t soff) {
    lds_dst = __builtin_amdgcn_readfirstlane(lds_dst);
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}

// acc += W-fragment x A-fragment with the scale byte pair SEL (0: bytes 0/1 of the slab's dword by
// half-wave, 2: bytes 2/3) of the shifted scale registers.  With BIT >= 0 the instruction is skipped when
// that bit of the wavefront-uniform `live` mask is clear; the branch sits inside the statement so that the
// compiler sees straight-line code and adds nothing between the scheduled instructions.
#define CMX_PIPE_MFMA(SELHI, EXTRA)                                                                             \
    if constexpr (BIT < 0)                                                                                      \
        asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:" SELHI EXTRA           \
                     : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));                                           \
    else                                                                                                        \
        asm volatile("s_bitcmp1_b32 %5, %6\n\ts_cbranch_scc0 .Lskip%=\n\t"                                      \
                     "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:" SELHI EXTRA           \
                     "\n.Lskip%=:"                                                                              \
                     : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live), "n"(BIT < 0 ? 0 : BIT) : "scc")
template <int FMT, int SEL, int BIT>
__device__ __forceinline__ void mfma_acc(v16f& acc, const v8i& w, const v8i& a, uint32_t sw, uint32_t sa, uint32_t live) {
    static_assert(SEL == 0 || SEL == 2, "scale byte pair");
    live = __builtin_amdgcn_readfirstlane(live);      // uniform by construction; makes it a scalar operand for certain
    if constexpr (FMT == CMX_FMT_E4M3) {
        if constexpr (SEL == 0) { CMX_PIPE_MFMA("[0,0,0]", ""); } else { CMX_PIPE_MFMA("[1,1,0]", ""); }
    } else {
        if constexpr (SEL == 0) { CMX_PIPE_MFMA("[0,0,0]", " cbsz:1 blgp:1"); } else { CMX_PIPE_MFMA("[1,1,0]", " cbsz:1 blgp:1"); }
    }
}
#undef CMX_PIPE_MFMA

// MFMA sequence of a step: the operand with more fragments runs in the outer loop (weights on a tie).  The
// fragments (0..FW-1 weights, FW..FW+FM-1 activations) are read in the order of their first use by it.
template <int FW, int FM>
__device__ __forceinline__ constexpr int pipe_read_order(int pos) {
    if (FM > FW) return pos == 0 ? FW : (pos <= FW ? pos - 1 : pos);          // A0 W0..W(FW-1) A1 A2 ...
    return pos == 0 ? 0 : (pos <= FM ? FW + pos - 1 : pos - FM);              // W0 A0..A(FM-1) W1 W2 ...
}

__device__ __forceinline__ v8i join8(const v4i& lo, const v4i& hi) {
    return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// Tile = 256 weight rows x TM activation rows, NSLOT ring slots of one slab each.
//   TM 256, 2 slots, WW x WM = 2 x 2: every wavefront owns a 128 x 128 corner (least LDS traffic per MFMA;
//           dense problems).
//   TM 256, 2 slots, 4 x 1: every wavefront owns 64 weight rows x all activation rows and skips the MFMAs of
//           the 32-row activation blocks past the tile's last valid row, so the last tile of a ragged group
//           costs what it holds (grouped problems).
//   TM 128, 3 slots, 4 x 1: two slabs instead of one in flight behind the one being consumed, for groups
//           so short that every tile streams its weights from HBM once and the load latency, not the MFMA
//           rate, sets the pace.
__host__ __device__ constexpr bool pipe_is_persistent(int nslot, int epi) { return nslot == 2 && epi != kEpiStore; }
// The persistent 2 x 2 kernels with the lean 16-bit store epilogue write their output in whole lines through an LDS
// staging area of 4 KiB per wavefront: the 16 KiB that the rings leave free, including the mailbox and the prefetch sink.
__host__ __device__ constexpr bool pipe_stages_stores(int nslot, int epi, int ww, int wm) {
    return pipe_is_persistent(nslot, epi) && epi_is_lean_store(epi) && ww == 2 && wm == 2;
}

// L2 prefetch distance in slabs for the persistent 2 x 2 kernels (0: none).  The workgroups that run side by side on
// an XCD share operand panels, and without help the one that is furthest ahead pays the HBM latency of every shared
// line for all of them.  While the load stream requests slab q, the workgroup therefore also touches one dword of
// every 128-byte line of slab q + distance -- of its share of the weight panel's rows: the m-tiles of a band share the
// panel, and each takes the rows congruent to its position in the band, so every line is asked for once per XCD, one
// to two slab times before the LDS-DMA loads of all sharers want it.  The loads have no register destination (they
// land in a 256-byte LDS sink nobody reads), and they are issued behind the tile loads of their slab, so every wait in
// the schedule simply lets two more loads stay in flight.  Loads return in order, so a prefetch must be back within
// about one and a half slab times or it holds up the tile loads behind it: distances 1 to 3 gain 4-5 % on the
// Zipf-routed 16-expert problem, 4 gains less, 10 nothing (the further ahead, the more often the line comes all the
// way from HBM).  The price is per distinct line: prefetching every line of the tile from every workgroup (512 lines per
// slab instead of 32) costs 20 %, and the activation panels, which only four workgroups share, lose more than they gain.
#ifndef CMX_PIPE_PREFETCH
#define CMX_PIPE_PREFETCH 2
#endif


template <int FMT, int EPI, int TM, int WW, int WM, int NSLOT>
__global__ __launch_bounds__(256) void mx_gemm_pipe_kernel(const GemmParams p) {
    static_assert(FMT == CMX_FMT_E4M3 || FMT == CMX_FMT_E5M2, "8-bit element formats only");
    static_assert((TM == 256 && NSLOT == 2 && ((WW == 2 && WM == 2) || (WW == 4 && WM == 1))) ||
                      (TM == 128 && NSLOT == 3 && WW == 4 && WM == 1), "tile / ring / wavefront layout");
    constexpr int TW = 256, NW = 4, FW = TW / WW / 32, FM = TM / WM / 32, NF = FW + FM;
    constexpr int kM = FW * FM;                                // MFMAs per step and wavefront (16 or 8)
    constexpr bool kMOuter = FM > FW;                          // activation fragment in the outer MFMA loop
    constexpr bool kSkip = WM == 1;
    constexpr int kRows = TW + TM;
    constexpr int kSlotBytes = kRows * kSlabBytes;            // 64 KiB or 48 KiB
    constexpr int kScaleBase = NSLOT * kSlotBytes;            // scale ring behind the tile slots
    // Two-slot kernels fetch the scales of FOUR slabs at a time (16 bytes per row, one load per 64 rows): a scale
    // load touches a different cache line in every lane, so one load per slab would pull as many lines through
    // the vector L1 as the tile data itself.  Their scale ring holds two such blocks, [block][row][4 dwords].
    // The three-slot kernel keeps one dword per row and slab, [slot][row].
    constexpr bool kSc4 = NSLOT == 2;
    constexpr int kScaleSlotBytes = kSc4 ? kRows * 16 : kRows * 4;
    constexpr int kScaleRingBytes = kSc4 ? 2 * kScaleSlotBytes : NSLOT * kScaleSlotBytes;
    constexpr int kTileLoads = kRows / (8 * NW);              // LDS-DMA loads per wavefront and slab (16 or 12)
    constexpr int kWTileLoads = TW / (8 * NW);                // the first 8 fetch weight rows
    constexpr int kLoadsPerSlab = kTileLoads + 2;             // three-slot kernel: plus one weight and one activation scale load
    constexpr int kPfAhead = (pipe_is_persistent(NSLOT, EPI) && WW == 2 && WM == 2) ? CMX_PIPE_PREFETCH : 0;
    constexpr int kPf = kPfAhead > 0 ? 2 : 0;                  // prefetch loads per wavefront and slab

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t ww = wave % WW, wm = wave / WW;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    // ---- tile sequence of this workgroup ------------------------------------------------------------------
    // The two-slot kernels with the SwiGLU or the lean 16-bit store epilogue are persistent: the grid is one
    // workgroup per CU, and workgroup j of XCD x walks tiles j, j + (workgroups per XCD), ... of that XCD's
    // contiguous run (or, in fixed strides over at least a round of tiles, the XCDs take turns at blocks of
    // consecutive tiles: interleave_xcd_walk), carrying the load pipeline across tile boundaries.  The others take one tile per
    // workgroup (the general store epilogue with its three output types and edge cases needs too many
    // registers to sit inside the loop).
    constexpr bool kPersistent = pipe_is_persistent(NSLOT, EPI);
    const uint32_t m_tiles_all = count_m_tiles<TM>(p);
    const uint32_t total_tiles = m_tiles_all * p.w_tiles;
    uint32_t run_count;
    const uint32_t run_first = xcd_run(total_tiles, blockIdx.x % kXcds, run_count);
    uint32_t run_end = run_first + run_count;
    uint32_t tile_stride = kPersistent ? gridDim.x / kXcds : total_tiles;      // one tile only when not persistent
    uint32_t tile_id = run_first + blockIdx.x / kXcds;
    if (kPersistent && p.tile_ctr == nullptr) interleave_xcd_walk(total_tiles, tile_id, tile_stride, run_end);
    if (!kPersistent && blockIdx.x < total_tiles) {
        tile_id = tile_of_workgroup(total_tiles);
        run_end = total_tiles;
    }
    if (tile_id >= run_end) return;

    // addressing of the tile whose slabs are being requested (switches two slabs before a tile boundary)
    Tile tq;                                    // tile of the load stream
    v4i w_rs, a_rs, ws_rs, as_rs;
    uint32_t goff[kTileLoads], sgoff_w, sgoff_a;
    uint32_t pfoff[2] = {0, 0};                 // prefetch: weight rows of this workgroup's share (wavefront 0; the others repeat one row)
    const uint32_t sa_blk = wave % (TM / 64);
    auto make_rsrc = [](const uint8_t* q) -> v4i {
        const uint64_t v = reinterpret_cast<uint64_t>(q);
        v4i r;
        r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));     // stride 0
        r[2] = -1;                                                           // no range limit
        r[3] = 0x00020000;
        return r;
    };
    auto aim_loads_at = [&](uint32_t L, uint32_t g_from) {
        decode_tile<TM>(p, m_tiles_all, L, tq, g_from);
        const uint32_t g = __builtin_amdgcn_readfirstlane(tq.g), wt = __builtin_amdgcn_readfirstlane(tq.wt);
        const uint32_t row0 = __builtin_amdgcn_readfirstlane(tq.row0);
        const uint32_t rows_valid = __builtin_amdgcn_readfirstlane(tq.rows_valid);
        tq.g = g; tq.wt = wt; tq.row0 = row0; tq.rows_valid = rows_valid;
        tq.mt = __builtin_amdgcn_readfirstlane(tq.mt);
        w_rs = make_rsrc(p.w + (size_t)g * p.n * p.ldw);
        ws_rs = make_rsrc(p.w_scale + (size_t)g * p.n * p.ld_ws);
        a_rs = make_rsrc(p.a + (size_t)row0 * p.lda);
        as_rs = make_rsrc(p.a_scale + (size_t)row0 * p.ld_as);
        // global row of tile row r (rows past the edge re-read the last valid row; their results are never stored)
        auto wrow_of = [&](uint32_t r) -> uint32_t {
            uint32_t gr;
            if (epi_is_swiglu_quant(EPI)) {
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
        // LDS-DMA load i of this wavefront fills combined tile rows (4i + wave)*8 .. +8; lane q -> row +q/8, LDS
        // chunk q%8, and fetches the global chunk that the XOR swizzle maps there
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) {
            const uint32_t cr = (NW * i + wave) * 8 + (lane >> 3);
            const uint32_t logical = swz(cr, lane & 7u);
            goff[i] = (i < kWTileLoads ? mul_lo_u32(wrow_of(cr), p.ldw) : mul_lo_u32(arow_of(cr - TW), p.lda)) + logical * 16;
        }
        // scale dwords: this wavefront fetches those of weight rows 64*wave.. and of activation rows
        // 64*(wave mod TM/64).. (with TM = 128 two wavefronts fetch the same rows to the same place)
        sgoff_w = wrow_of(64 * wave + lane) * p.ld_ws;
        sgoff_a = arow_of(64 * sa_blk + lane) * p.ld_as;
        if constexpr (kPf > 0) {
            static_assert(kPf == 0 || (TW == 256 && TM == 256), "the prefetch split assumes 256 + 256 rows");
            // The workgroups that run side by side on an XCD share operand panels (tile order: bands of m-tiles, m
            // fastest, across a run of weight tiles): the weight panel with the other m-tiles of the band.  Each
            // prefetches only its share of the panel's rows (row = position in the band, modulo the band's height);
            // the lanes left over repeat the last such row.
            const uint32_t band = p.row_off != nullptr ? 8u : 4u;
            const uint32_t mtg = p.row_off != nullptr ? (uint32_t)table_at(p.tile_pref, g + 1) - (uint32_t)table_at(p.tile_pref, g) : m_tiles_all;
            const uint32_t mt = tq.mt, b0 = mt / band * band;
            const uint32_t mod = __builtin_amdgcn_readfirstlane(mtg - b0 < band ? mtg - b0 : band);      // m-tiles that share the weight panel
            const uint32_t sel = __builtin_amdgcn_readfirstlane(mt - b0);
            const uint32_t last = __builtin_amdgcn_readfirstlane(sel + mod * ((255u - sel) / mod));
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                // Weight panels only, and only when at least three m-tiles of the band share one: on the 16-expert problem
                // the weight panels (up to eight sharers) gain 4.3 % alone, the activation panels (four weight tiles side
                // by side) lose 1.7 % alone, both together gain 3.6 %; thresholds of 3 / 5 / 6 / 8 sharers for the weight
                // panels: 855.6 / 859.4 / 861.1 / 869.3 us.  Dense problems, whose workgroups run in lock step, lose 1-2 %.
                // At most 86 rows: the two loads of wavefront 0 cover them, every other lane repeats the last one.
                uint32_t r = sel + mod * (j * 64 + lane);
                r = (r < 256u && wave == 0 && mod >= 3u && p.row_off != nullptr) ? r : last;
                pfoff[j] = mul_lo_u32(wrow_of(r), p.ldw);
            }
        }
    };
    aim_loads_at(tile_id, 0);
    Tile tc = tq;                               // tile of the MFMA stream / epilogue

    auto nslab_of = [](const GemmParams& q) -> uint32_t { return q.kbytes / kSlabBytes; };
    const uint32_t nslab = nslab_of(p);
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    constexpr int kScaleRowBytes = kSc4 ? 16 : 4;
    const uint32_t sdma_base = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + wave * 64 * kScaleRowBytes);
    const uint32_t sdma_base_a = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + (TW + sa_blk * 64) * kScaleRowBytes);

    auto issue_tile_load = [&](int slot, int i, uint32_t koff) {
        dma_b128(dma_base + slot * kSlotBytes + i * (NW * 1024), goff[i], i < kWTileLoads ? w_rs : a_rs, koff);
    };
    const uint32_t pf_sink = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + kScaleRingBytes + 256);
    auto issue_prefetch = [&](int j, uint32_t koff) { dma_b32(pf_sink, pfoff[j], w_rs, koff); };
    auto issue_scale_loads = [&](int slot, uint32_t soff) {          // one slab (three-slot kernel)
        dma_b32(sdma_base + slot * kScaleSlotBytes, sgoff_w, ws_rs, soff);
        dma_b32(sdma_base_a + slot * kScaleSlotBytes, sgoff_a, as_rs, soff);
    };
    // four slabs: block `blk` of the load stream's tile into ring position `pos` (0/1)
    uint32_t blocks_issued = 0;          // running count over all tiles of this workgroup: ring position = count & 1
    auto issue_scale_block = [&](uint32_t blk) {
        const uint32_t pos = blocks_issued & 1u;
        ++blocks_issued;
        dma_b128(sdma_base + pos * kScaleSlotBytes, sgoff_w, ws_rs, blk * 16);
        dma_b128(sdma_base_a + pos * kScaleSlotBytes, sgoff_a, as_rs, blk * 16);
    };
    // the load stream is at slab q of its tile: block 0 goes out with slab 0, block b+1 with slab 4b+1 (the ring
    // position it takes was last read one slab earlier)
    const uint32_t nblk = nslab_of(p) / 4;
    auto scale_block_due = [&](uint32_t q) -> bool { return q == 0 || ((q & 3u) == 1u && (q >> 2) + 1 < nblk); };
    auto scale_block_of = [&](uint32_t q) -> uint32_t { return q == 0 ? 0u : (q >> 2) + 1; };
    auto clamp_slab = [&](uint32_t slab) -> uint32_t { return slab < nslab ? slab : nslab - 1; };   // past the end: harmless reload

    // ---- fragment read addresses ------------------------------------------------------------------
    // a lane reads 16-byte chunks lh, lh+2 (step 0) and lh+4, lh+6 (step 1) of its row; all rows of a
    // lane share the low five bits l32, hence the swizzle term
    const uint32_t x = (l32 & 7u) ^ ((l32 >> 3) & 1u);
    const uint32_t w_row_base = epi_is_swiglu_quant(EPI) ? ww * (TW / 2 / WW) : ww * (TW / WW);
    uint32_t wb[NSLOT][4], ab[NSLOT][4];       // [slot][chunk j]
#pragma unroll
    for (int s = 0; s < NSLOT; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t ch = ((lh + 2 * j) ^ x) * 16;
            wb[s][j] = lds0 + s * kSlotBytes + (w_row_base + l32) * kSlabBytes + ch;
            ab[s][j] = lds0 + s * kSlotBytes + (TW + wm * (TM / WM) + l32) * kSlabBytes + ch;
        }
    const uint32_t swb = lds0 + kScaleBase + (w_row_base + l32) * kScaleRowBytes;
    const uint32_t sab = lds0 + kScaleBase + (TW + wm * (TM / WM) + l32) * kScaleRowBytes;
    // two-slot kernels: running index (over all tiles) of the slab whose scales are read next; its block sits
    // at ring position (index / 4) & 1, its dword at index & 3
    uint32_t scale_read_slab = 0;
    auto scale_read_offset = [&]() -> uint32_t {
        return __builtin_amdgcn_readfirstlane(((scale_read_slab >> 2) & 1u) * kScaleSlotBytes + (scale_read_slab & 3u) * 4);
    };
    const uint32_t sshift = 8 * lh;

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // fragment sets: index 0..FW-1 weights, FW.. activations; lo = registers 0-3, hi = registers 4-7
    v4i f0lo[NF], f0hi[NF], f1lo[NF], f1hi[NF];
    uint32_t sraw[NF], scur[NSLOT][NF];      // shifted scales alternate between two sets: a set is rewritten one slab after its last use

    // weight fragment f sits f*32 rows (SwiGLU: the gate fragments, then their up partners 128 rows on) below the base
#define CMX_PIPE_WOFF(f) ((epi_is_swiglu_quant(EPI) ? ((f) < FW / 2 ? (f) * 32 : TW / 2 + ((f) - FW / 2) * 32) : (f) * 32))
    // one 16-byte read: r = 2 * position in the read order + half (0: registers 0-3, 1: registers 4-7)
    // The two-slot grouped kernels (persistent 2 x 2, and 4 x 1) read the step-1 fragments weights first: the weight rows of a
    // slot are then free a few MFMAs into step 0 (four with 2 x 2 wavefronts, two with 4 x 1, whose wavefronts hold only two
    // weight fragments), a barrier says so, and the eight weight loads of slab s+2 -- the ones that come from HBM -- go out
    // five to six MFMAs earlier than the slot as a whole would allow, while the activation fragments are still being read.
    // 0.7 % on the 16-expert problem (2 x 2), 3.2 % on GMM1 of the 256-expert FFN (4 x 1, private weight panels streamed
    // from HBM).  Three or four reads per MFMA to free the rows earlier still: slower.
    constexpr bool kWFirst = kPf > 0 || (kSkip && NSLOT == 2);
    auto read_half = [&](auto slot_c, auto step_c, auto r_c, v4i (&flo)[NF], v4i (&fhi)[NF]) {
        constexpr int slot = decltype(slot_c)::value, step = decltype(step_c)::value, r = decltype(r_c)::value;
        constexpr int idx = (kWFirst && step == 1) ? r / 2 : pipe_read_order<FW, FM>(r / 2), half = r % 2;
        (void)wb, (void)ab;
        v4i& dst = half ? fhi[idx] : flo[idx];
        if constexpr (idx < FW) dst = lds_read_b128<CMX_PIPE_WOFF(idx) * kSlabBytes>(wb[slot][2 * step + half]);
        else dst = lds_read_b128<(idx - FW) * 32 * kSlabBytes>(ab[slot][2 * step + half]);
    };
    auto read_frag = [&](auto slot_c, auto step_c, auto idx_c, v4i (&flo)[NF], v4i (&fhi)[NF]) {     // by position in the read order
        constexpr int pos = decltype(idx_c)::value;
        read_half(slot_c, step_c, std::integral_constant<int, 2 * pos>{}, flo, fhi);
        read_half(slot_c, step_c, std::integral_constant<int, 2 * pos + 1>{}, flo, fhi);
    };
    auto read_scale = [&](auto slot_c, auto idx_c) {                 // three-slot kernel: [slot][row]
        constexpr int slot = decltype(slot_c)::value, idx = decltype(idx_c)::value;
        if constexpr (idx < FW)
            sraw[idx] = lds_read_b32<slot * kScaleSlotBytes + CMX_PIPE_WOFF(idx) * 4>(swb);
        else
            sraw[idx] = lds_read_b32<slot * kScaleSlotBytes + (idx - FW) * 32 * 4>(sab);
    };
    // two-slot kernels: swb_at / sab_at = base + ring position and dword of the slab being read
    auto read_scale_at = [&](uint32_t swb_at, uint32_t sab_at, auto idx_c) {
        constexpr int idx = decltype(idx_c)::value;
        (void)sraw;
        if constexpr (idx < FW)
            sraw[idx] = lds_read_b32<CMX_PIPE_WOFF(idx) * 16>(swb_at);
        else
            sraw[idx] = lds_read_b32<(idx - FW) * 32 * 16>(sab_at);
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;

    // ---- prologue: fill the ring, wait for slab 0 -------------------------------------------------------
    if constexpr (kSc4) {
        // scale blocks first, so that the wait below can leave exactly the 16 tile loads of slab 1 in flight
        issue_scale_block(0);
        if (nblk > 1) issue_scale_block(1);
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) issue_tile_load(0, i, 0);
        const uint32_t k1 = clamp_slab(1);
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) issue_tile_load(1, i, k1 * kSlabBytes);
        if constexpr (kPf > 0) {
            const uint32_t kp = clamp_slab(1 + kPfAhead) * kSlabBytes;
            issue_prefetch(0, kp);
            issue_prefetch(1, kp);
        }
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kTileLoads + kPf) : "memory");      // slab 0 and its scales have landed everywhere
        static_for<0, NF>([&](auto ic) { read_frag(I0{}, I0{}, ic, f0lo, f0hi); });
        {
            const uint32_t off = scale_read_offset();
            const uint32_t swb_at = swb + off, sab_at = sab + off;
            static_for<0, NF>([&](auto ic) { read_scale_at(swb_at, sab_at, ic); });
            ++scale_read_slab;
        }
    } else {
        static_for<0, NSLOT>([&](auto sc) {
            constexpr int slot = decltype(sc)::value;
            const uint32_t k = clamp_slab(slot);
#pragma unroll
            for (int i = 0; i < kTileLoads; ++i) issue_tile_load(slot, i, k * kSlabBytes);
            issue_scale_loads(slot, k * 4);
        });
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NSLOT - 1) * kLoadsPerSlab) : "memory");      // slab 0 has landed everywhere
        static_for<0, NF>([&](auto ic) { read_frag(I0{}, I0{}, ic, f0lo, f0hi); });
        static_for<0, NF>([&](auto ic) { read_scale(I0{}, ic); });
    }

    auto shift_scales = [&](auto set_c) {
        constexpr int set = decltype(set_c)::value;
        (void)scur, (void)sraw, (void)sshift;      // asm operands alone do not make a generic lambda capture
#pragma unroll
        for (int i = 0; i < NF; ++i) asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(scur[set][i]) : "v"(sshift), "v"(sraw[i]));
        asm volatile("s_nop 1" ::: "memory");      // the next MFMA may be the very next instruction (skipped ones in between)
    };
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    shift_scales(I0{});

    // activation blocks of 32 rows that hold valid rows (4 x 1 layout: the others are skipped)
    auto live_mask = [](uint32_t rows_valid) -> uint32_t { return __builtin_amdgcn_readfirstlane((1u << ((rows_valid + 31) / 32)) - 1u); };
    uint32_t live = live_mask(tc.rows_valid);      // bit fm: block fm has valid rows
    auto step_mfma = [&](auto sel_c, auto i_c, v4i (&flo)[NF], v4i (&fhi)[NF], auto set_c) {
        constexpr int sel = decltype(sel_c)::value, i = decltype(i_c)::value, set = decltype(set_c)::value;
        constexpr int fw = kMOuter ? i % FW : i / FM, fm = kMOuter ? i / FW : i % FM;
        (void)scur, (void)acc;
        mfma_acc<FMT, sel, kSkip ? fm : -1>(acc[fw][fm], join8(flo[fw], fhi[fw]), join8(flo[FW + fm], fhi[FW + fm]), scur[set][fw],
                                            scur[set][FW + fm], live);
    };
    // A fragment set stays allocated to the end of the step that consumes it: the reads of the next set must
    // not be given a register that an MFMA issued a few cycles earlier may still be fetching.
    auto pin_fragments = [&](v4i (&flo)[NF], v4i (&fhi)[NF]) {
#pragma unroll
        for (int i = 0; i < NF; ++i) asm volatile("" ::"v"(flo[i]), "v"(fhi[i]));
    };
    // Keep a slab's scale registers allocated to the end of the slab: otherwise the shifts for the next slab
    // may be given the register of a scale whose last reader is an MFMA issued a few cycles earlier, and
    // nothing orders that VALU write behind the MFMA's operand fetch.
    auto pin_scales = [&](auto set_c) {
        constexpr int set = decltype(set_c)::value;
        (void)scur;
#pragma unroll
        for (int i = 0; i < NF; ++i) asm volatile("" ::"v"(scur[set][i]));
    };
    constexpr int kReads = 2 * NF;
    constexpr uint32_t kNoSlab = 0xFFFFFFFFu;

    // ---- two-slot ring -------------------------------------------------------------------------------------
    // One slab; SLOT = ring slot of slab s (compile-time so that every LDS offset is an immediate).  On entry
    // fragment set 0 and the shifted scales of the slab are in registers.  kR reads go behind each of the first
    // MFMAs of a step; after MFMA kB1 the last of them has had time to land; kEarly tile loads of slab s+2
    // are issued already in step 0, behind the first barrier.
    // q = slab of the load stream within its tile (kNoSlab: nothing new to request, re-request slab koff)
    // kpf = byte offset of the slab to prefetch (two-by-two persistent kernels)
    auto slab_body2 = [&](auto slot_c, uint32_t koff, uint32_t q, uint32_t kpf) {
        constexpr int slot = decltype(slot_c)::value;
        constexpr int kR = NF > 8 ? 3 : 2;
        constexpr int kB1 = (kReads + kR - 1) / kR;
        constexpr int kEarly = kM - kB1 - 1;
        constexpr int kScaleMfmas = (NF + 1) / 2;              // MFMAs that carry two scale reads each
        static_assert(kM == 16 && kB1 + kScaleMfmas + 1 <= 14, "the scale shift must sit at least two MFMAs before the end of the step");
        using SlotT = std::integral_constant<int, slot>;
        using OtherT = std::integral_constant<int, slot ^ 1>;
        const uint32_t sc_off = scale_read_offset();             // where the scales of the next slab sit
        const uint32_t swb_at = swb + sc_off, sab_at = sab + sc_off;
        ++scale_read_slab;
        // ---- step 0 ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I0{}, ic, f0lo, f0hi, SlotT{});
            static_for<0, kR>([&](auto jc) {
                constexpr int r = i * kR + decltype(jc)::value;
                if constexpr (r < kReads) read_half(SlotT{}, I1{}, std::integral_constant<int, r>{}, f1lo, f1hi);
            });
            if constexpr (kWFirst) {
                // the weight rows of slot `slot` have been read for the last time (fragments 0..FW-1, kR halves per MFMA):
                // once everyone is here they can be refilled, while the activation rows are still being read
                constexpr int kBw = (2 * FW + kR - 1) / kR - 1;
                if constexpr (i == kBw) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                if constexpr (i > kBw && i - kBw - 1 < kWTileLoads) issue_tile_load(slot, i - kBw - 1, koff);
                if constexpr (i == kB1) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            } else {
            // slot `slot` has been read for the last time: once everyone is here it can be refilled
            if constexpr (i == kB1) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if constexpr (i > kB1) issue_tile_load(slot, i - kB1 - 1, koff);
            }
        });
        pin_fragments(f0lo, f0hi);
        // own loads of slab s+1 are complete (only the kEarly loads just issued may be in flight); after the
        // barrier so are everyone's
        constexpr int kEarlyN = kWFirst ? kWTileLoads : kEarly;
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kEarlyN + kPf) : "memory");
        // ---- step 1 ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I2{}, ic, f1lo, f1hi, SlotT{});
            if constexpr (i + kEarlyN < kTileLoads) issue_tile_load(slot, i + kEarlyN, koff);
            if constexpr (i + kEarlyN == kTileLoads) {
                if (q != kNoSlab && scale_block_due(q)) issue_scale_block(scale_block_of(q));
            }
            static_for<0, kR>([&](auto jc) {
                constexpr int r = i * kR + decltype(jc)::value;
                if constexpr (r < kReads) read_half(OtherT{}, I0{}, std::integral_constant<int, r>{}, f0lo, f0hi);
            });
            if constexpr (i >= kB1 && i < kB1 + kScaleMfmas) {
                read_scale_at(swb_at, sab_at, std::integral_constant<int, 2 * (i - kB1)>{});
                if constexpr (2 * (i - kB1) + 1 < NF) read_scale_at(swb_at, sab_at, std::integral_constant<int, 2 * (i - kB1) + 1>{});
            }
            if constexpr (i == kB1 + kScaleMfmas + 1) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                shift_scales(OtherT{});
            }
            // behind every tile load and the scale block of this slab: the waits above count on that order
            if constexpr (kPf > 0 && i == kB1 + kScaleMfmas) issue_prefetch(0, kpf);
            if constexpr (kPf > 0 && i == kB1 + kScaleMfmas + 2) issue_prefetch(1, kpf);
        });
        pin_fragments(f1lo, f1hi);
        pin_scales(SlotT{});
    };

    // ---- three-slot ring (8 MFMAs per step) -----------------------------------------------------------------
    // While slab s (slot s%3) is consumed, slab s+1 is landing or landed and slab s+2 is in flight.  Half way
    // through, everybody has read slot s%3 for the last time and waited for its own loads of slab s+1: one
    // barrier frees the slot and publishes slab s+1, and the loads of slab s+3 go straight into the freed
    // slot, so two slabs are in flight for two slab times each.
    auto slab_body3 = [&](auto slot_c, uint32_t s) {
        constexpr int slot = decltype(slot_c)::value;
        static_assert(NSLOT == 2 || (kM == 8 && kReads == 12 && kTileLoads == 12 && NF == 6), "three-slot schedule is written for the 256 x 128 tile");
        using SlotT = std::integral_constant<int, slot>;
        using NextT = std::integral_constant<int, (slot + 1) % 3>;
        const uint32_t k3 = clamp_slab(s + 3);
        const uint32_t koff = k3 * kSlabBytes, soff = k3 * 4;
        // ---- step 0: second half of the slab into fragment set 1 ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I0{}, ic, f0lo, f0hi, SlotT{});
            if constexpr (2 * i < kReads) {
                read_half(SlotT{}, I1{}, std::integral_constant<int, 2 * i>{}, f1lo, f1hi);
                read_half(SlotT{}, I1{}, std::integral_constant<int, 2 * i + 1>{}, f1lo, f1hi);
            }
        });
        pin_fragments(f0lo, f0hi);
        // own reads of slot `slot` and own loads of slab s+1 are complete (slab s+2 may be in flight)
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kLoadsPerSlab) : "memory");
        // ---- step 1: loads of slab s+3 into the freed slot, first half of slab s+1 into fragment set 0 ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I2{}, ic, f1lo, f1hi, SlotT{});
            if constexpr (i < 3) {                 // the six scale dwords first: they are waited for before the fragments
                read_scale(NextT{}, std::integral_constant<int, 2 * i>{});
                read_scale(NextT{}, std::integral_constant<int, 2 * i + 1>{});
            }
            if constexpr (2 * i < kTileLoads) {
                issue_tile_load(slot, 2 * i, koff);
                issue_tile_load(slot, 2 * i + 1, koff);
            }
            if constexpr (2 * i == kTileLoads) issue_scale_loads(slot, soff);
            if constexpr (2 * i < kReads) {
                read_half(NextT{}, I0{}, std::integral_constant<int, 2 * i>{}, f0lo, f0hi);
                read_half(NextT{}, I0{}, std::integral_constant<int, 2 * i + 1>{}, f0lo, f0hi);
            }
            if constexpr (i == 6) {
                // LDS reads return in order, and 8 fragment reads (two of MFMA 2, all of MFMAs 3..5) were issued
                // after the last scale read: the scales are in once at most those 8 are outstanding
                asm volatile("s_waitcnt lgkmcnt(8)" ::: "memory");
                shift_scales(NextT{});
            }
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // fragment set 0 of the next slab
        pin_fragments(f1lo, f1hi);
        pin_scales(SlotT{});
    };

    // The compiler does not see the MFMAs inside the asm statements, so it inserts none of the wait states
    // that separate them from its own accumulator accesses.  Passing every accumulator through an asm
    // statement that holds the wait states pins those accesses to the far side of it.
    auto fence_accumulators = [&]() {
        v16f* const a = &acc[0][0];
        asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]), "+a"(a[4]), "+a"(a[5]), "+a"(a[6]), "+a"(a[7]));
        if constexpr (kM == 16)
            asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[8]), "+a"(a[9]), "+a"(a[10]), "+a"(a[11]), "+a"(a[12]), "+a"(a[13]), "+a"(a[14]), "+a"(a[15]));
    };
    fence_accumulators();       // the zero initialisation has retired before the first MFMA reads it
    if constexpr (NSLOT == 3) {
        uint32_t s = 0;
        for (; s + 3 <= nslab; s += 3) {
            slab_body3(I0{}, s);
            slab_body3(I1{}, s + 1);
            slab_body3(I2{}, s + 2);
        }
        const uint32_t rem = nslab - s;                 // the ring position after whole turns is slot 0 again
        if (rem >= 1) slab_body3(I0{}, s);
        if (rem == 2) slab_body3(I1{}, s + 1);
        // the loads issued past the end must land before the LDS is released; the last MFMAs must have
        // written their accumulators before the epilogue reads them
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        fence_accumulators();
        epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
    } else if constexpr (!kPersistent) {
        for (uint32_t s = 0; s < nslab; s += 2) {      // the host only selects this kernel for a slab count that is a multiple of four
            const uint32_t q0 = s + 2, q1 = s + 3;
            slab_body2(I0{}, clamp_slab(q0) * kSlabBytes, q0 < nslab ? q0 : kNoSlab, 0);
            slab_body2(I1{}, clamp_slab(q1) * kSlabBytes, q1 < nslab ? q1 : kNoSlab, 0);
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        fence_accumulators();
        epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
    } else {
        // The host only selects this kernel for a slab count that is a multiple of four.  The load stream runs two slabs ahead of
        // the MFMA stream: when it reaches the end of the tile it is aimed at the workgroup's next tile (or keeps
        // re-requesting the last slab when there is none), so the loads and the fragment reads run on through
        // the tile boundary and only the epilogue and the clearing of the accumulators interrupt the MFMAs.
        // One loop holds every case so that the register assignment of the scheduled part never changes.
        // Next tile: with a counter array (grouped problems in the 4 x 1 layout, whose tiles differ in cost) the workgroups of an
        // XCD draw from that XCD's run in order; without one the walk is strided.
        uint32_t sm = 0;             // slab of the MFMA stream within its tile
        uint32_t sq = 2;             // slab of the load stream within its tile
        bool next_ok = false;        // the load stream has moved on to a next tile
        uint32_t next_id = tile_id;
        for (;;) {
            if (sq == nslab) {
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
                    aim_loads_at(next_id, tq.g);      // tile ids only grow
                    sq = 0;
                }
            }
            slab_body2(I0{}, clamp_slab(sq) * kSlabBytes, sq < nslab ? sq : kNoSlab, clamp_slab(sq + kPfAhead) * kSlabBytes);
            slab_body2(I1{}, clamp_slab(sq + 1) * kSlabBytes, sq + 1 < nslab ? sq + 1 : kNoSlab, clamp_slab(sq + 1 + kPfAhead) * kSlabBytes);
            sq += 2;
            sm += 2;
            if (sm == nslab) {
                fence_accumulators();           // the last MFMAs have written their accumulators
                if constexpr (pipe_stages_stores(NSLOT, EPI, WW, WM)) {
                    // The staging area overlays the sink of the prefetch loads: every wavefront's loads must have landed
                    // before anyone stages.  (They are the next tile's first two slabs and their prefetches, issued a slab
                    // ago.)  No prefetch is issued again before two barriers of the next slab, when everyone is done here.
                    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
                    lean_store_lines<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane, lds0 + kScaleBase + kScaleRingBytes + wave * 4096);
                } else {
                    epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
                }
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
                // The last slab has already read the new tile's first fragments and scales, but carrying them
                // through the epilogue costs more registers than there are: read them again (slot 0, landed).
                static_for<0, NF>([&](auto ic) { read_frag(I0{}, I0{}, ic, f0lo, f0hi); });
                {
                    --scale_read_slab;          // the slab whose scales the last body read: the new tile's slab 0
                    const uint32_t off = scale_read_offset();
                    const uint32_t swb_at = swb + off, sab_at = sab + off;
                    static_for<0, NF>([&](auto ic) { read_scale_at(swb_at, sab_at, ic); });
                    ++scale_read_slab;
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                shift_scales(I0{});
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // the re-requested slabs land before the LDS is released
    }
#undef CMX_PIPE_WOFF
}
