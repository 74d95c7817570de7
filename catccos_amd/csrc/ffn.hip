// Single-device MoE FFN: routing sort -> fused quantise+scatter -> GMM1 (+SwiGLU +requant) ->
// GMM2 -> weighted combine, chained on one stream with no host synchronisation.
#include "mx_common.h"

namespace cmx {
namespace {

constexpr size_t kAlign = 512;

// The reference operator's published workspace size for the same arguments (512-byte aligned
// regions: row index, bf16 dispatch staging, metadata, quantised rows + scales, SwiGLU staging,
// requantised rows + scales, bf16 return staging, metadata).
size_t reference_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t experts, uint32_t top_k) {
    const size_t rows = (size_t)m * top_k;
    const size_t meta = (size_t)experts * sizeof(int32_t);
    auto al = [](size_t b) { return round_up_sz(b, kAlign); };
    const size_t ready = (size_t)experts * 64;
    const size_t swiglu_staging = rows * (n / 2) * 2;
    const size_t dispatch_ready = round_up_sz((size_t)experts * 4, 64) + ready;
    const size_t dispatch_staging = rows * k * 2;
    return al(round_up_sz(m, 256) * top_k * sizeof(int32_t)) + al(rows * k * 2) + al(meta) + al(rows * k) +
           al(rows * scale_cols(k)) + al(swiglu_staging > ready ? swiglu_staging : ready) + al(rows * (n / 2)) +
           al(rows * scale_cols(n / 2)) + al(dispatch_staging > dispatch_ready ? dispatch_staging : dispatch_ready) +
           al(meta);
}

void layout(uint32_t m, uint32_t k, uint32_t n, uint32_t experts, uint32_t top_k, cmx_ffn_workspace_layout* L) {
    const size_t rows = (size_t)m * top_k;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += round_up_sz(bytes ? bytes : 1, kAlign);
        return at;
    };
    L->src2sorted = take(rows * 4);
    L->sorted2src = take(rows * 4);
    L->counts = take((size_t)experts * 4);
    L->routing_scratch = take(cmx_moe_routing_workspace_bytes((uint32_t)rows, experts));
    L->gmm_meta = take(2 * cmx_mx_gmm_workspace_bytes(experts));
    L->a_codes = take(rows * k);
    // scale rows of the dispatched tokens at a pitch of whole 128-byte lines: the scatter then writes every line of
    // this array whole
    L->a_scales_pitch = round_up(scale_cols(k), 128);
    L->a_scales = take(rows * (size_t)L->a_scales_pitch);
    L->act_codes = take(rows * (n / 2));
    L->act_scales = take(rows * scale_cols(n / 2));
    L->y = take(rows * k * 2);
    const size_t ref = reference_workspace_bytes(m, k, n, experts, top_k);
    L->total = off > ref ? off : ref;
}

}  // namespace
}  // namespace cmx

extern "C" uint64_t catccos_ascend950_symmetric_bytes(void) { return 1004ull * 1024 * 1024; }

extern "C" int cmx_ffn_workspace_layout_get(uint32_t m, uint32_t k, uint32_t n, uint32_t localExperts, uint32_t topK,
                                            cmx_ffn_workspace_layout* out) {
    using namespace cmx;
    CMX_REQUIRE(out, "null pointer");
    CMX_REQUIRE(m > 0 && k > 0 && n > 0 && localExperts > 0 && topK > 0, "shape must be positive");
    layout(m, k, n, localExperts, topK, out);
    return CMX_OK;
}

extern "C" size_t catccos_ascend950_dispatch_ffn_combine_workspace_bytes(uint32_t m, uint32_t k, uint32_t n,
                                                                         uint32_t localExperts, uint32_t topK,
                                                                         int rankSize) {
    if (rankSize != 1 || m == 0 || k == 0 || n == 0 || localExperts == 0 || topK == 0) return 0;
    cmx_ffn_workspace_layout L;
    cmx::layout(m, k, n, localExperts, topK, &L);
    return L.total;
}

namespace cmx {
namespace {
int ffn_chain(cmx_stream_t stream, const uint8_t* x, const uint8_t* expertIdx, const uint8_t* gateWeight, const uint8_t* w1,
              const uint8_t* w1Scale, const uint8_t* w2, const uint8_t* w2Scale, uint8_t* out, uint8_t* workspace, uint32_t m,
              uint32_t k, uint32_t n, uint32_t localExperts, uint32_t topK, bool pretiled) {
    CMX_REQUIRE(x && expertIdx && gateWeight && w1 && w1Scale && w2 && w2Scale && out && workspace, "null pointer");
    CMX_REQUIRE(m > 0 && localExperts > 0 && topK > 0 && topK <= localExperts, "bad routing shape");
    // limits of the stages further down the chain, checked before anything is launched
    CMX_REQUIRE(topK <= 64, "topK must not exceed 64 (weighted combine)");
    CMX_REQUIRE((uint64_t)m * topK < (1ull << 31), "m * topK must stay below 2^31 routes");
    CMX_REQUIRE(k % 256 == 0 && n % 512 == 0, "MXFP8 FFN requires K % 256 == 0 and N % 512 == 0");
    CMX_REQUIRE(!pretiled || (k % 512 == 0 && n % 1024 == 0), "pre-tiled weights require K % 512 == 0 and N % 1024 == 0");
    CMX_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0, "workspace must be 256-byte aligned");
    cmx_ffn_workspace_layout L;
    layout(m, k, n, localExperts, topK, &L);
    const uint32_t rows = m * topK;
    int32_t* src2sorted = reinterpret_cast<int32_t*>(workspace + L.src2sorted);
    int32_t* sorted2src = reinterpret_cast<int32_t*>(workspace + L.sorted2src);
    int32_t* counts = reinterpret_cast<int32_t*>(workspace + L.counts);
    uint8_t* a_codes = workspace + L.a_codes;
    uint8_t* a_scales = workspace + L.a_scales;
    uint8_t* act_codes = workspace + L.act_codes;
    uint8_t* act_scales = workspace + L.act_scales;
    uint8_t* y = workspace + L.y;
    uint8_t* meta1 = workspace + L.gmm_meta;
    uint8_t* meta2 = meta1 + cmx_mx_gmm_workspace_bytes(localExperts);

    int rc = cmx_moe_init_routing(reinterpret_cast<const int32_t*>(expertIdx), m, topK, localExperts, sorted2src,
                                  src2sorted, counts, workspace + L.routing_scratch, stream);
    if (rc != CMX_OK) return rc;
    const uint32_t ld_as = (uint32_t)L.a_scales_pitch;
    rc = cmx_quant_scatter(x, k, src2sorted, a_codes, k, a_scales, ld_as, m, k, topK, stream);
    if (rc != CMX_OK) return rc;
    const uint32_t ld_acts = scale_cols(n / 2);
    rc = pretiled ? cmx_mx_gmm_swiglu_quant_pretiled(a_codes, k, a_scales, ld_as, w1, w1Scale, act_codes, n / 2, act_scales,
                                                     ld_acts, nullptr, counts, localExperts, rows, n, k, meta1, stream)
                  : cmx_mx_gmm_swiglu_quant(a_codes, k, a_scales, ld_as, w1, w1Scale, act_codes, n / 2, act_scales, ld_acts,
                                            nullptr, counts, localExperts, rows, n, k, meta1, stream);
    if (rc != CMX_OK) return rc;
    rc = pretiled ? cmx_mx_gmm_pretiled(act_codes, n / 2, act_scales, ld_acts, w2, w2Scale, y, k, counts, localExperts, rows, k,
                                        n / 2, CMX_FMT_E4M3, CMX_OUT_BF16, meta2, stream)
                  : cmx_mx_gmm(act_codes, n / 2, act_scales, ld_acts, w2, w2Scale, y, k, counts, localExperts, rows, k, n / 2,
                               CMX_FMT_E4M3, CMX_OUT_BF16, meta2, stream);
    if (rc != CMX_OK) return rc;
    return cmx_moe_token_unpermute(y, k, rows, src2sorted, reinterpret_cast<const float*>(gateWeight), out, k, m, k,
                                   topK, stream);
}
}  // namespace
}  // namespace cmx

extern "C" int catccos_ascend950_dispatch_ffn_combine(uint32_t blockDim, cmx_stream_t stream, uint64_t fftsAddr,
                                                      const uint8_t* x, const uint8_t* expertIdx,
                                                      const uint8_t* gateWeight, const uint8_t* w1,
                                                      const uint8_t* w1Scale, const uint8_t* w2, const uint8_t* w2Scale,
                                                      uint8_t* out, uint8_t* workspace, uint8_t* symmetric, uint32_t m,
                                                      uint32_t k, uint32_t n, uint32_t localExperts, uint32_t topK,
                                                      int rankSize) {
    using namespace cmx;
    (void)blockDim;
    (void)fftsAddr;
    (void)symmetric;
    CMX_REQUIRE(rankSize == 1, "one device only: rankSize must be 1");
    return ffn_chain(stream, x, expertIdx, gateWeight, w1, w1Scale, w2, w2Scale, out, workspace, m, k, n, localExperts, topK,
                     false);
}

extern "C" int cmx_dispatch_ffn_combine_pretiled(cmx_stream_t stream, const uint8_t* x, const uint8_t* expertIdx,
                                                 const uint8_t* gateWeight, const uint8_t* w1_tiled, const uint8_t* w1Scale,
                                                 const uint8_t* w2_tiled, const uint8_t* w2Scale, uint8_t* out,
                                                 uint8_t* workspace, uint32_t m, uint32_t k, uint32_t n,
                                                 uint32_t localExperts, uint32_t topK) {
    return cmx::ffn_chain(stream, x, expertIdx, gateWeight, w1_tiled, w1Scale, w2_tiled, w2Scale, out, workspace, m, k, n,
                          localExperts, topK, true);
}
