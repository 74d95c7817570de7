// Hand-scheduled 256 x 256 block-scaled matmul kernel for MXFP4 (E2M1, two codes per byte), included by
// mx_gemm.hip after mx_gemm_pipe.h, whose helpers and conventions it shares.
//
// A 128-byte K slab holds 256 FP4 elements = four MFMA steps of 64 K; a lane's fragment of one step is a
// single 16-byte run (the 32-element MX block of its half-wave), and a slab carries two scale dwords per
// row.  As in the 8-bit two-slot kernels the scales arrive 16 bytes per row at a time -- here the scales of two
// slabs -- into a ring of two such blocks, [block][row][4 dwords].  An FP4 MFMA takes 8 passes (32 clocks), so a
// slab is again 64 x 32 = 2048 MFMA clocks per wavefront for the same 64 KiB of loads as in the 8-bit kernel, but
// an MFMA leaves room for only about six other instructions: the instruction stream is kept thin (a load's M0
// write and the load itself stand on either side of an MFMA instead of an s_nop, both scale dwords of a row come
// with one 8-byte read, the byte shifts are spread over a step).  Four wavefronts, 16 accumulator tiles in AGPRs,
// two fragment sets of NF x 4 VGPRs.  Per slab s (ring slot s%2):
//   step 0:    16 MFMAs; behind the first NF the reads of step 1's fragments, behind the others the scale reads
//              of slab s+1 (its block landed long ago);
//   step 1:    behind the first NF MFMAs the reads of step 2's fragments, behind the others the per-half-wave
//              byte shifts of those scales into the other scale set;
//   step 2:    reads of step 3; after MFMA 9 they have landed and the slot is never read again: barrier, then the
//              first 6 tile loads of slab s+2 around the remaining MFMAs; the step ends with the wait for the own
//              loads of slab s+1 and the barrier that publishes it;
//   step 3:    the other 10 tile loads of slab s+2 (and, every second slab, the next scale block) and the reads of
//              step 0 of slab s+1 from the other slot.
// With the lean 16-bit store epilogues the kernel is persistent like its 8-bit counterpart: one workgroup per CU
// walks the tiles of its XCD's run and carries the load stream across tile boundaries, so that the first slabs of
// a tile arrive while the previous tile's epilogue runs.  With the general store epilogue it takes one tile per
// workgroup.
#pragma once

// An LDS-DMA load in two statements, so that a scheduled instruction (an MFMA, an LDS read) can stand where the wait
// state between the write of M0 and the load would otherwise be an s_nop.  Nothing between the two may write M0.
__device__ __forceinline__ void dma_aim(uint32_t lds_dst) {
    lds_dst = __builtin_amdgcn_readfirstlane(lds_dst);
    asm volatile("s_mov_b32 m0, %0" ::"s"(lds_dst) : "memory");
}
__device__ __forceinline__ void dma_b128_aimed(uint32_t voff, v4i rsrc, uint32_t soff) {
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void dma_b32_aimed(uint32_t voff, v4i rsrc, uint32_t soff) {
    soff = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("buffer_load_dword %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
typedef int v2i __attribute__((ext_vector_type(2)));
template <int OFF>
__device__ __forceinline__ v2i lds_read_b64(uint32_t addr) {
    v2i r;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}

template <int SEL, int BIT>
__device__ __forceinline__ void mfma_acc_fp4(v16f& acc, const v4i& w, const v4i& a, uint32_t sw, uint32_t sa, uint32_t live) {
    static_assert(SEL == 0 || SEL == 2, "scale byte pair");
    live = __builtin_amdgcn_readfirstlane(live);
    if constexpr (BIT < 0) {
        if constexpr (SEL == 0)
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
        else
            asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[1,1,0] cbsz:4 blgp:4"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa));
    } else {
        if constexpr (SEL == 0)
            asm volatile("s_bitcmp1_b32 %5, %6\n\ts_cbranch_scc0 .Lskip%=\n\t"
                         "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4\n.Lskip%=:"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live), "n"(BIT < 0 ? 0 : BIT) : "scc");
        else
            asm volatile("s_bitcmp1_b32 %5, %6\n\ts_cbranch_scc0 .Lskip%=\n\t"
                         "v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[1,1,0] cbsz:4 blgp:4\n.Lskip%=:"
                         : "+a"(acc) : "v"(w), "v"(a), "v"(sw), "v"(sa), "s"(live), "n"(BIT < 0 ? 0 : BIT) : "scc");
    }
}

// WW x WM = 2 x 2 (dense) or 4 x 1 (grouped: skips the MFMAs of activation blocks without valid rows)
template <int EPI, int WW, int WM>
__global__ __launch_bounds__(256) void mx_gemm_pipe_fp4_kernel(const GemmParams p) {
    static_assert((WW == 2 && WM == 2) || (WW == 4 && WM == 1), "wavefront layout");
    static_assert(!epi_pairs_gate_up(EPI), "store epilogues only");
    constexpr int TW = 256, TM = 256, NW = 4, FW = TW / WW / 32, FM = TM / WM / 32, NF = FW + FM;
    constexpr int kM = FW * FM;                                // 16 MFMAs per step and wavefront
    constexpr bool kMOuter = FM > FW;
    constexpr bool kSkip = WM == 1;
    constexpr int kRows = TW + TM;
    constexpr int kSlotBytes = kRows * kSlabBytes;            // 64 KiB
    constexpr int kScaleBase = 2 * kSlotBytes;
    constexpr int kScaleSlotBytes = kRows * 16;               // one block: 16 bytes (the scales of two slabs) per row
    constexpr int kTileLoads = kRows / (8 * NW);              // 16
    constexpr int kWTileLoads = TW / (8 * NW);
    static_assert(kM == 16 && NF + NF / 2 < kM, "schedule is written for 16 MFMAs per step");
    // L2 prefetch of the persistent 2 x 2 kernels, as in mx_gemm_pipe_kernel: two loads per wavefront and slab
    constexpr int kPfAhead = (pipe_is_persistent(2, EPI) && WW == 2 && WM == 2) ? CMX_PIPE_PREFETCH : 0;
    constexpr int kPf = kPfAhead > 0 ? 2 : 0;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t ww = wave % WW, wm = wave / WW;
    const uint32_t l32 = lane & 31u, lh = lane >> 5;

    // ---- tile sequence of this workgroup (see mx_gemm_pipe_kernel) ----
    constexpr bool kPersistent = pipe_is_persistent(2, EPI);
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
    Tile tq;
    v4i w_rs, a_rs, ws_rs, as_rs;
    uint32_t goff[kTileLoads], sgoff_w, sgoff_a;
    uint32_t pfoff[2] = {0, 0};                 // prefetch: weight rows of this workgroup's share (wavefront 0; the others repeat one row)
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
            const uint32_t gr = wt * TW + r;
            return gr < p.n ? gr : p.n - 1;
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
        sgoff_w = wrow_of(64 * wave + lane) * p.ld_ws;
        sgoff_a = arow_of(64 * wave + lane) * p.ld_as;
        if constexpr (kPf > 0) {
            // each workgroup prefetches its share of the weight panel it has in common with the other m-tiles of its band
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

    const uint32_t nslab = p.kbytes / kSlabBytes;
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const uint32_t sdma_base = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + wave * 64 * 16);
    const uint32_t sdma_base_a = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + (TW + wave * 64) * 16);

    auto issue_tile_load = [&](int slot, int i, uint32_t slab) {
        dma_b128(dma_base + slot * kSlotBytes + i * (NW * 1024), goff[i], i < kWTileLoads ? w_rs : a_rs, slab * kSlabBytes);
    };
    // the same in two halves, with an MFMA between them
    auto aim_tile_load = [&](int slot, int i) { dma_aim(dma_base + slot * kSlotBytes + i * (NW * 1024)); };
    auto fire_tile_load = [&](int i, uint32_t slab) { dma_b128_aimed(goff[i], i < kWTileLoads ? w_rs : a_rs, slab * kSlabBytes); };
    const uint32_t pf_sink = __builtin_amdgcn_readfirstlane(lds0 + kScaleBase + 2 * kScaleSlotBytes + 256);
    // block `blk` of the load stream's tile (the scales of its slabs 2 blk and 2 blk + 1) into the next ring position
    const uint32_t nblk = nslab / 2;
    uint32_t blocks_issued = 0;          // running count over all tiles of this workgroup: ring position = count & 1
    auto issue_scale_block = [&](uint32_t blk) {
        const uint32_t pos = blocks_issued & 1u;
        ++blocks_issued;
        dma_b128(sdma_base + pos * kScaleSlotBytes, sgoff_w, ws_rs, blk * 16);
        dma_b128(sdma_base_a + pos * kScaleSlotBytes, sgoff_a, as_rs, blk * 16);
    };
    // the load stream is at slab q of its tile: block 0 goes out with slab 0, block b with slab 2b - 1 (the ring
    // position it takes was last read one slab earlier)
    auto scale_block_due = [&](uint32_t q) -> bool { return q == 0 || ((q & 1u) && (q + 1) / 2 < nblk); };
    auto scale_block_of = [&](uint32_t q) -> uint32_t { return (q + 1) / 2; };
    auto clamp_slab = [&](uint32_t slab) -> uint32_t { return slab < nslab ? slab : nslab - 1; };   // past the end: harmless reload

    // fragment read addresses: step h reads the 16-byte chunk 2h + lh of the lane's row
    const uint32_t x = (l32 & 7u) ^ ((l32 >> 3) & 1u);
    const uint32_t w_row_base = epi_pairs_gate_up(EPI) ? ww * (TW / 2 / WW) : ww * (TW / WW);
    uint32_t wb[2][4], ab[2][4];       // [slot][step]
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const uint32_t ch = ((2 * h + lh) ^ x) * 16;
            wb[s][h] = lds0 + s * kSlotBytes + (w_row_base + l32) * kSlabBytes + ch;
            ab[s][h] = lds0 + s * kSlotBytes + (TW + wm * (TM / WM) + l32) * kSlabBytes + ch;
        }
    const uint32_t swb = lds0 + kScaleBase + (w_row_base + l32) * 16;
    const uint32_t sab = lds0 + kScaleBase + (TW + wm * (TM / WM) + l32) * 16;
    const uint32_t sshift = 8 * lh;

    v16f acc[FW][FM];
#pragma unroll
    for (int i = 0; i < FW; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    v4i fa[NF], fb[NF];                 // the two fragment sets: 0..FW-1 weights, FW.. activations
    v2i sraw[NF];                       // the two scale dwords of a slab, as read
    uint32_t scur[2][2][NF];            // shifted: [ring slot][dword of the slab][fragment]

#define CMX_PIPE_WOFF(f) ((epi_pairs_gate_up(EPI) ? ((f) < FW / 2 ? (f) * 32 : TW / 2 + ((f) - FW / 2) * 32) : (f) * 32))
    auto read_piece = [&](auto slot_c, auto step_c, auto pos_c, v4i (&f)[NF]) {
        constexpr int slot = decltype(slot_c)::value, step = decltype(step_c)::value;
        // the last step's fragments of a slot are read weights first in the grouped kernels, so that the weight rows
        // are free (and their loads go out) while the activation fragments are still being read
        constexpr int idx = ((kPf > 0 || kSkip) && step == 3) ? decltype(pos_c)::value : pipe_read_order<FW, FM>(decltype(pos_c)::value);
        (void)wb, (void)ab;
        if constexpr (idx < FW) f[idx] = lds_read_b128<CMX_PIPE_WOFF(idx) * kSlabBytes>(wb[slot][step]);
        else f[idx] = lds_read_b128<(idx - FW) * 32 * kSlabBytes>(ab[slot][step]);
    };
    // both dwords of the slab whose scales sit at swb_at / sab_at (= base + ring position + 8 * (slab & 1))
    auto read_scale = [&](uint32_t swb_at, uint32_t sab_at, auto idx_c) {
        constexpr int idx = decltype(idx_c)::value;
        (void)sraw;
        if constexpr (idx < FW)
            sraw[idx] = lds_read_b64<CMX_PIPE_WOFF(idx) * 16>(swb_at);
        else
            sraw[idx] = lds_read_b64<(idx - FW) * 32 * 16>(sab_at);
    };
    // running index (over all tiles) of the slab whose scales are read next: its block sits at ring position
    // (index / 2) & 1, its two dwords at 8 * (index & 1)
    uint32_t scale_read_slab = 0;
    auto scale_read_offset = [&]() -> uint32_t {
        return __builtin_amdgcn_readfirstlane(((scale_read_slab >> 1) & 1u) * kScaleSlotBytes + (scale_read_slab & 1u) * 8);
    };
    // per-half-wave byte shift of fragment idx's scales into set `set`
    auto shift_scale = [&](auto set_c, auto idx_c) {
        constexpr int set = decltype(set_c)::value, i = decltype(idx_c)::value;
        (void)scur, (void)sraw, (void)sshift;
        asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(scur[set][0][i]) : "v"(sshift), "v"(sraw[i][0]));
        asm volatile("v_lshrrev_b32 %0, %1, %2" : "=v"(scur[set][1][i]) : "v"(sshift), "v"(sraw[i][1]));
    };
    auto pin_fragments = [&](v4i (&f)[NF]) {
#pragma unroll
        for (int i = 0; i < NF; ++i) asm volatile("" ::"v"(f[i]));
    };
    auto pin_scales = [&](auto set_c) {
        constexpr int set = decltype(set_c)::value;
        (void)scur;
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int i = 0; i < NF; ++i) asm volatile("" ::"v"(scur[set][d][i]));
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;

    // ---- prologue ------------------------------------------------------------------------------------------
    // scale blocks first, so that the wait below can leave exactly the tile loads of slab 1 in flight
    issue_scale_block(0);
    if (nblk > 1) issue_scale_block(1);
#pragma unroll
    for (int i = 0; i < kTileLoads; ++i) issue_tile_load(0, i, 0);
    {
        const uint32_t k1 = clamp_slab(1);
#pragma unroll
        for (int i = 0; i < kTileLoads; ++i) issue_tile_load(1, i, k1);
    }
    if constexpr (kPf > 0) {
        const uint32_t kp = clamp_slab(1 + kPfAhead) * kSlabBytes;
        dma_b32(pf_sink, pfoff[0], w_rs, kp);
        dma_b32(pf_sink, pfoff[1], w_rs, kp);
    }
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kTileLoads + kPf) : "memory");      // slab 0 and its scales have landed everywhere
    // step 0 of the slab in slot 0 and its scales into fragment set a / scale set 0
    auto read_first_step = [&]() {
        static_for<0, NF>([&](auto ic) { read_piece(I0{}, I0{}, ic, fa); });
        const uint32_t off = scale_read_offset();
        const uint32_t swb_at = swb + off, sab_at = sab + off;
        static_for<0, NF>([&](auto ic) { read_scale(swb_at, sab_at, ic); });
        ++scale_read_slab;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        static_for<0, NF>([&](auto ic) { shift_scale(I0{}, ic); });
        asm volatile("s_nop 1" ::: "memory");      // the first MFMA may be the very next instruction
    };
    read_first_step();

    auto live_mask = [](uint32_t rows_valid) -> uint32_t { return __builtin_amdgcn_readfirstlane((1u << ((rows_valid + 31) / 32)) - 1u); };
    uint32_t live = live_mask(tc.rows_valid);      // bit fm: activation block fm has valid rows
    // step h of the slab in ring slot `set`: scale dword h/2, byte pair 2*(h%2)
    auto step_mfma = [&](auto h_c, auto i_c, v4i (&f)[NF], auto set_c) {
        constexpr int h = decltype(h_c)::value, i = decltype(i_c)::value, set = decltype(set_c)::value;
        constexpr int fw = kMOuter ? i % FW : i / FM, fm = kMOuter ? i / FW : i % FM;
        (void)scur, (void)acc;
        mfma_acc_fp4<(h & 1) * 2, kSkip ? fm : -1>(acc[fw][fm], f[fw], f[FW + fm], scur[set][h >> 1][fw], scur[set][h >> 1][FW + fm], live);
    };

    constexpr int kB1 = 9;                      // MFMA of step 2 after which the reads of step 3 have landed
    constexpr int kEarly = kM - kB1 - 1;        // tile loads of slab s+2 issued in step 2 (6)
    constexpr bool kWFirst = kPf > 0 || kSkip;  // grouped kernels: the eight weight loads go out early instead (see read_piece)
    constexpr int kEarlyN = kWFirst ? kWTileLoads : kEarly;
    constexpr uint32_t kNoSlab = 0xFFFFFFFFu;
    // q = slab of the load stream within its tile (kNoSlab: nothing new to request, slab q2 is requested again)
    // qpf = slab to prefetch (persistent 2 x 2 kernels)
    auto slab_body = [&](auto slot_c, uint32_t q2, uint32_t q, uint32_t qpf) {
        constexpr int slot = decltype(slot_c)::value;
        using SlotT = std::integral_constant<int, slot>;
        using OtherT = std::integral_constant<int, slot ^ 1>;
        const uint32_t sc_off = scale_read_offset();             // where the scales of the next slab sit
        const uint32_t swb_at = swb + sc_off, sab_at = sab + sc_off;
        ++scale_read_slab;
        // ---- step 0: fragments of step 1; behind them the scales of the next slab (they landed long ago) ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I0{}, ic, fa, SlotT{});
            if constexpr (i < NF) read_piece(SlotT{}, I1{}, ic, fb);
            if constexpr (i >= NF && 2 * (i - NF) < NF) {
                read_scale(swb_at, sab_at, std::integral_constant<int, 2 * (i - NF)>{});
                if constexpr (2 * (i - NF) + 1 < NF) read_scale(swb_at, sab_at, std::integral_constant<int, 2 * (i - NF) + 1>{});
            }
        });
        pin_fragments(fa);
        asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NF) : "memory");        // LDS reads return in order: all but the NF scale reads
        // ---- step 1: fragments of step 2; then the byte shifts of the next slab's scales ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            step_mfma(I1{}, ic, fb, SlotT{});
            if constexpr (i < NF) read_piece(SlotT{}, I2{}, ic, fa);
            if constexpr (i == NF) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NF) : "memory");      // the scale reads, not the NF fragment reads behind them
            if constexpr (i >= NF) {
                constexpr int per = (NF + (kM - NF) - 1) / (kM - NF);          // fragments per MFMA
                static_for<0, per>([&](auto jc) {
                    constexpr int idx = (i - NF) * per + decltype(jc)::value;
                    if constexpr (idx < NF) shift_scale(OtherT{}, std::integral_constant<int, idx>{});
                });
            }
        });
        pin_fragments(fb);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // ---- step 2: last reads of the slot, first loads of slab s+2 ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (kWFirst) {
                // weight fragments 0..FW-1 are read behind MFMAs 0..FW-1: behind MFMA FW the weight rows of the slot are free
                if constexpr (i > FW && i - FW - 1 < kWTileLoads) aim_tile_load(slot, i - FW - 1);
                step_mfma(I2{}, ic, fa, SlotT{});
                if constexpr (i < NF) read_piece(SlotT{}, I3{}, ic, fb);
                if constexpr (i == FW) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                if constexpr (i > FW && i - FW - 1 < kWTileLoads) fire_tile_load(i - FW - 1, q2);
                if constexpr (i == kB1) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            } else {
                if constexpr (i > kB1) aim_tile_load(slot, i - kB1 - 1);
                step_mfma(I2{}, ic, fa, SlotT{});
                if constexpr (i < NF) read_piece(SlotT{}, I3{}, ic, fb);
                if constexpr (i == kB1) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                if constexpr (i > kB1) fire_tile_load(i - kB1 - 1, q2);
            }
        });
        pin_fragments(fa);
        // own loads of slab s+1 are complete (only the early loads just issued may be in flight); after the
        // barrier so are everyone's
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(kEarlyN + kPf) : "memory");
        // ---- step 3: the other loads, the first fragments of the next slab ----
        static_for<0, kM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            if constexpr (i + kEarlyN < kTileLoads) aim_tile_load(slot, i + kEarlyN);
            // the prefetch loads go behind every tile load and the scale block of this slab: the waits count on that order
            if constexpr (kPf > 0 && (i == kTileLoads - kEarlyN + 2 || i == kTileLoads - kEarlyN + 4)) dma_aim(pf_sink);
            step_mfma(I3{}, ic, fb, SlotT{});
            if constexpr (i < NF) read_piece(OtherT{}, I0{}, ic, fa);
            if constexpr (i + kEarlyN < kTileLoads) fire_tile_load(i + kEarlyN, q2);
            if constexpr (i + kEarlyN == kTileLoads) {
                if (q != kNoSlab && scale_block_due(q)) issue_scale_block(scale_block_of(q));
            }
            if constexpr (kPf > 0 && i == kTileLoads - kEarlyN + 2) dma_b32_aimed(pfoff[0], w_rs, qpf * kSlabBytes);
            if constexpr (kPf > 0 && i == kTileLoads - kEarlyN + 4) dma_b32_aimed(pfoff[1], w_rs, qpf * kSlabBytes);
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      // fragment set a of the next slab
        pin_fragments(fb);
        pin_scales(SlotT{});
    };

    // The compiler does not see the MFMAs inside the asm statements: every accumulator passes through an asm
    // statement that holds the wait states between them and the compiler's own accumulator accesses.
    auto fence_accumulators = [&]() {
        v16f* const a = &acc[0][0];
        asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[0]), "+a"(a[1]), "+a"(a[2]), "+a"(a[3]), "+a"(a[4]), "+a"(a[5]), "+a"(a[6]), "+a"(a[7]));
        asm volatile("s_nop 15\n\ts_nop 15" : "+a"(a[8]), "+a"(a[9]), "+a"(a[10]), "+a"(a[11]), "+a"(a[12]), "+a"(a[13]), "+a"(a[14]), "+a"(a[15]));
    };
    fence_accumulators();       // the zero initialisation has retired before the first MFMA reads it
    if constexpr (!kPersistent) {
        for (uint32_t s = 0; s < nslab; s += 2) {      // the host only selects this kernel for an even slab count
            const uint32_t q0 = s + 2, q1 = s + 3;
            slab_body(I0{}, clamp_slab(q0), q0 < nslab ? q0 : kNoSlab, 0);
            slab_body(I1{}, clamp_slab(q1), q1 < nslab ? q1 : kNoSlab, 0);
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        fence_accumulators();
        epilogue<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane);
    } else {
        // The load stream runs two slabs ahead of the MFMA stream: at the end of a tile it is aimed at the
        // workgroup's next tile (or keeps requesting the last slab again when there is none).  With a counter
        // array (grouped problems) the workgroups of an XCD draw their next tile from that XCD's run in order.
        uint32_t sm = 0;             // slab of the MFMA stream within its tile
        uint32_t sq = 2;             // slab of the load stream within its tile
        bool next_ok = false;        // the load stream has moved on to a next tile
        uint32_t next_id = tile_id;
        for (;;) {
            if (sq == nslab) {
                if (p.tile_ctr != nullptr) {
                    uint32_t* const mailbox = reinterpret_cast<uint32_t*>(smem + kScaleBase + 2 * kScaleSlotBytes);
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
            slab_body(I0{}, clamp_slab(sq), sq < nslab ? sq : kNoSlab, clamp_slab(sq + kPfAhead));
            slab_body(I1{}, clamp_slab(sq + 1), sq + 1 < nslab ? sq + 1 : kNoSlab, clamp_slab(sq + 1 + kPfAhead));
            sq += 2;
            sm += 2;
            if (sm == nslab) {
                fence_accumulators();           // the last MFMAs have written their accumulators
                if constexpr (pipe_stages_stores(2, EPI, WW, WM)) {
                    // whole-line stores through the staging area that overlays the prefetch sink (see mx_gemm_pipe_kernel)
                    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
                    lean_store_lines<TW, TM, WW, WM, EPI, FW, FM>(p, tc, acc, ww, wm, lane, lds0 + kScaleBase + 2 * kScaleSlotBytes + wave * 4096);
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
                // the last slab body has read the new tile's first fragments and scales already; they are not
                // carried through the epilogue but read again (slot 0, landed)
                --scale_read_slab;
                read_first_step();
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");     // the re-requested slabs land before the LDS is released
    }
#undef CMX_PIPE_WOFF
}
