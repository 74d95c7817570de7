// Single-instruction probes of the block-scaled MFMA, used by the register-layout known-answer
// tests: the caller supplies every lane's operand registers and scale register verbatim.
#include "mx_common.h"

namespace cmx {
namespace {

template <int FMTCODE, int SEL>
__global__ void raw_probe_32(const v8i* a, const v8i* b, const int* sa, const int* sb, v16f* out) {
    const int t = threadIdx.x;
    v16f acc;
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[t], b[t], acc, FMTCODE, FMTCODE, SEL, sa[t], SEL, sb[t]);
    out[t] = acc;
}

template <int FMTCODE, int SEL>
__global__ void raw_probe_16(const v8i* a, const v8i* b, const int* sa, const int* sb, v4f* out) {
    const int t = threadIdx.x;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[t], b[t], acc, FMTCODE, FMTCODE, SEL, sa[t], SEL, sb[t]);
    out[t] = acc;
}

template <int FMTCODE>
int launch_probe(int shape, int sel, hipStream_t s, const void* a, const void* b, const int* sa, const int* sb,
                 void* out) {
#define CMX_PROBE(SEL)                                                                                         \
    if (shape == 0)                                                                                            \
        hipLaunchKernelGGL((raw_probe_32<FMTCODE, SEL>), dim3(1), dim3(64), 0, s, (const v8i*)a, (const v8i*)b, sa, \
                           sb, (v16f*)out);                                                                    \
    else                                                                                                       \
        hipLaunchKernelGGL((raw_probe_16<FMTCODE, SEL>), dim3(1), dim3(64), 0, s, (const v8i*)a, (const v8i*)b, sa, \
                           sb, (v4f*)out);
    switch (sel) {
        case 0: CMX_PROBE(0) break;
        case 1: CMX_PROBE(1) break;
        case 2: CMX_PROBE(2) break;
        default: CMX_PROBE(3) break;
    }
#undef CMX_PROBE
    CMX_LAUNCH_CHECK();
    return CMX_OK;
}

}  // namespace
}  // namespace cmx

// a_regs/b_regs: int32 [64 lanes][8]; sa/sb: int32 [64]; out: fp32 [64][16] (shape 0: 32x32x64) or
// [64][4] (shape 1: 16x16x128).  opsel selects the scale byte for both operands.
extern "C" int cmx_mfma_raw_probe(const void* a_regs, const void* b_regs, const int32_t* sa, const int32_t* sb,
                                  float* out, int fmt, int opsel, int shape, cmx_stream_t stream) {
    using namespace cmx;
    CMX_REQUIRE(a_regs && b_regs && sa && sb && out, "null pointer");
    CMX_REQUIRE(opsel >= 0 && opsel < 4 && (shape == 0 || shape == 1), "bad selector");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (fmt) {
        case CMX_FMT_E4M3: return launch_probe<0>(shape, opsel, s, a_regs, b_regs, sa, sb, out);
        case CMX_FMT_E5M2: return launch_probe<1>(shape, opsel, s, a_regs, b_regs, sa, sb, out);
        case CMX_FMT_E2M1: return launch_probe<4>(shape, opsel, s, a_regs, b_regs, sa, sb, out);
        default: set_error("cmx_mfma_raw_probe: unknown element format"); return CMX_EINVAL;
    }
}
