// "DispatchGmmDequantSwiglu" on one GPU: route tokens to experts, quantise + scatter them, grouped matmul
// with the gate|up weights, dequant, SwiGLU.  Two arithmetics, chosen with Arithmetic():
//  * kInt8 - the reference operator itself (examples/dispatch_gmm_dequant_swiglu/
//    dispatch_gmm_dequant_swiglu_host.h:18-125): per-token dynamic INT8 activations, INT8 weights [E, K, N],
//    per-channel scales in 64-bit words, bf16 output [m * topK, n / 2]; the reference's buffer order
//    (A = x, B = weights, C = out, custom = { scale, expertIdx }) and .bin names.
//  * kMx (default) - the same chain restated in MXFP8 (examples/utils/gen_data_moe.py:628-658 up to the requant),
//    with an MX requant of the result.
#ifndef DISPATCH_GMM_DEQUANT_SWIGLU_HOST_H
#define DISPATCH_GMM_DEQUANT_SWIGLU_HOST_H

#include "op_common.h"

class DispatchGmmDequantSwigluOperator : public CatccosOperator {
public:
    enum { kMx = 0, kInt8 = 1 };
    static int& Arithmetic() { static int a = kMx; return a; }

    // ---- INT8 (the reference operator's own arithmetic) ------------------------------------------------
    struct Int8Layout {
        size_t src2sorted, sorted2src, routing, counts, aCodes, tokScale, gmm, total;
    };
    static Int8Layout Int8WorkspaceLayout(const CocTilingParams& t)
    {
        const uint32_t experts = t.expertNum / (t.epSize ? t.epSize : 1);
        const size_t rows = static_cast<size_t>(t.m) * t.topK;
        Int8Layout l{};
        size_t off = 0;
        auto take = [&](size_t b) { size_t at = off; off += RoundUp<size_t>(b ? b : 1, 512); return at; };
        l.src2sorted = take(rows * 4);
        l.sorted2src = take(rows * 4);
        l.routing = take(cmx_moe_routing_workspace_bytes(static_cast<uint32_t>(rows), experts));
        l.counts = take(experts * sizeof(int32_t));
        l.aCodes = take(rows * t.k);
        l.tokScale = take(rows * sizeof(float));
        l.gmm = take(cmx_int8_gmm_workspace_bytes(experts, t.n, t.k, 1));
        l.total = off;
        return l;
    }
    void AllocateInt8(KernelParams& params, const CocTilingParams& t, uint32_t rankId, const std::string& dataFile)
    {
        const size_t experts = t.expertNum / t.epSize;
        const size_t rows = static_cast<size_t>(t.m) * t.topK;
        const bool fromFiles = !dataFile.empty();
        auto file = [&](const char* stem) { return mxops::RankFile(dataFile, stem, rankId, false); };
        const size_t aBytes = static_cast<size_t>(t.m) * t.k * sizeof(uint16_t);
        uint8_t* a = nullptr;
        if (fromFiles) {
            a = mxops::DeviceBufferFromFile(aBytes, file("a_gm"));
        } else {
            std::vector<uint16_t> ones(static_cast<size_t>(t.m) * t.k, 0x3F80);
            a = mxops::DeviceBufferFromValues(ones.data(), aBytes);
        }
        // b_gm is [E, k, n] on disk; the weights do not change between launches, so they are rewritten K-contiguous
        // ([E, n, k]) once here and every launch runs with trans_b = 1 (otherwise each call would move them again)
        uint8_t* bFile = mxops::DeviceBufferFromFile(static_cast<size_t>(t.k) * t.n * experts, fromFiles ? file("b_gm") : "", 1);
        uint8_t* b = mxrt::DeviceAlloc(static_cast<size_t>(t.k) * t.n * experts);
        MX_CHECK(cmx_bytes_to_k_major(bFile, t.n, b, t.k, t.k, t.n, static_cast<uint32_t>(experts), nullptr));
        MX_CHECK(cmx_rt_stream_sync(nullptr));
        MX_CHECK(cmx_rt_free(bFile));
        uint8_t* scale = nullptr;
        const size_t scaleBytes = static_cast<size_t>(t.n) * experts * sizeof(uint64_t);
        if (fromFiles) {
            scale = mxops::DeviceBufferFromFile(scaleBytes, file("scale_gm"));
        } else {
            std::vector<uint64_t> words(static_cast<size_t>(t.n) * experts, 0x3F800000ull);      // fp32 1.0 in the low half
            scale = mxops::DeviceBufferFromValues(words.data(), scaleBytes);
        }
        uint8_t* expertIdx = nullptr;
        if (fromFiles) {
            expertIdx = mxops::DeviceBufferFromFile(rows * sizeof(int32_t), file("expert_idx"));
        } else {
            std::vector<int32_t> rr(rows);
            for (size_t i = 0; i < rows; ++i) rr[i] = static_cast<int32_t>(i % experts);
            expertIdx = mxops::DeviceBufferFromValues(rr.data(), rows * sizeof(int32_t));
        }
        uint8_t* c = mxops::DeviceBufferFromFile(rows * (t.n / 2) * sizeof(uint16_t), "", 0);
        params.SetKernelParams(a, b, c, scale, expertIdx);
    }
    static int LaunchInt8(void* stream, const KernelParams& p, uint8_t* ws, const CocTilingParams& t)
    {
        const Int8Layout l = Int8WorkspaceLayout(t);
        const uint32_t experts = t.expertNum / t.epSize;
        const uint32_t rows = t.m * t.topK;
        int32_t* src2sorted = reinterpret_cast<int32_t*>(ws + l.src2sorted);
        int32_t* counts = reinterpret_cast<int32_t*>(ws + l.counts);
        int rc = cmx_moe_init_routing(reinterpret_cast<const int32_t*>(p.customPtrs[1]), t.m, t.topK, experts,
                                      reinterpret_cast<int32_t*>(ws + l.sorted2src), src2sorted, counts, ws + l.routing, stream);
        if (rc != CMX_OK) return rc;
        int8_t* aCodes = reinterpret_cast<int8_t*>(ws + l.aCodes);
        float* tokScale = reinterpret_cast<float*>(ws + l.tokScale);
        rc = cmx_int8_quant_scatter(p.ptrA, t.k, src2sorted, aCodes, t.k, tokScale, t.m, t.k, t.topK, stream);
        if (rc != CMX_OK) return rc;
        return cmx_int8_gmm_dequant_swiglu(aCodes, t.k, tokScale, reinterpret_cast<const int8_t*>(p.ptrB),
                                           reinterpret_cast<const float*>(p.customPtrs[0]), 2, p.ptrC, t.n / 2, CMX_OUT_BF16, counts,
                                           experts, rows, t.n, t.k, 1, ws + l.gmm, stream);
    }

    // ---- MX ---------------------------------------------------------------------------------------------
    // ptrA = x bf16 [m,k], ptrB = W1 [E,n,k], ptrC = act codes E4M3 [m*topK, n/2],
    // custom = { expertIdx i32 [m,topK], W1 scale [E,n,k/32], act scales [m*topK, n/64], tokens per expert i32 [E] }
    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        if (Arithmetic() == kInt8) {
            AllocateInt8(params, t, rankId, dataFile);
            return;
        }
        const size_t experts = t.expertNum / t.epSize;
        const size_t rows = static_cast<size_t>(t.m) * t.topK;
        const size_t half = t.n / 2;
        const bool fromFiles = !dataFile.empty();
        auto file = [&](const char* stem) { return mxops::RankFile(dataFile, stem, rankId, false); };
        uint8_t* x = nullptr;
        const size_t xBytes = static_cast<size_t>(t.m) * t.k * sizeof(uint16_t);
        if (fromFiles) {
            x = mxops::DeviceBufferFromFile(xBytes, file("in_routing_matrix_a"));
        } else {
            std::vector<uint16_t> ones(static_cast<size_t>(t.m) * t.k, 0x3F80);
            x = mxops::DeviceBufferFromValues(ones.data(), xBytes);
        }
        uint8_t* w1 = mxops::DeviceBufferFromFile(static_cast<size_t>(t.k) * t.n * experts, fromFiles ? file("in_gmm_matrix_b") : "", 0x38);
        uint8_t* w1Scale = mxops::DeviceBufferFromFile(mxops::ScaleCols(t.k) * t.n * experts, fromFiles ? file("in_gmm_matrix_b_scale") : "", 120);
        uint8_t* expertIdx = nullptr;
        if (fromFiles) {
            expertIdx = mxops::DeviceBufferFromFile(rows * sizeof(int32_t), file("in_routing_expert_idx"));
        } else {
            std::vector<int32_t> rr(rows);
            for (size_t i = 0; i < rows; ++i) rr[i] = static_cast<int32_t>(i % experts);     // round-robin routing
            expertIdx = mxops::DeviceBufferFromValues(rr.data(), rows * sizeof(int32_t));
        }
        uint8_t* act = mxrt::DeviceAlloc(rows * half);
        uint8_t* actScale = mxrt::DeviceAlloc(rows * mxops::ScaleCols(half));
        uint8_t* counts = mxrt::DeviceAlloc(experts * sizeof(int32_t));
        params.SetKernelParams(x, w1, act, expertIdx, w1Scale, actScale, counts);
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t rows = static_cast<size_t>(t.m) * t.topK;
        const size_t half = t.n / 2;
        if (Arithmetic() == kInt8) {
            mxops::DeviceBufferToFile(params.ptrC, rows * half * sizeof(uint16_t), mxops::RankFile(dataFile, "output", rankId, false));
            return;
        }
        mxops::DeviceBufferToFile(params.ptrC, rows * half, mxops::RankFile(dataFile, "out_swiglu_quant", rankId, false));
        mxops::DeviceBufferToFile(params.customPtrs[2], rows * mxops::ScaleCols(half), mxops::RankFile(dataFile, "out_swiglu_scale", rankId, false));
        mxops::DeviceBufferToFile(params.customPtrs[3], (t.expertNum / t.epSize) * sizeof(int32_t), mxops::RankFile(dataFile, "out_routing_tokens", rankId, false));
    }

    struct Layout {
        size_t src2sorted, sorted2src, routing, meta, aCodes, aScales, total;
    };
    static Layout WorkspaceLayout(const CocTilingParams& t)
    {
        const uint32_t experts = t.expertNum / (t.epSize ? t.epSize : 1);
        const size_t rows = static_cast<size_t>(t.m) * t.topK;
        Layout l{};
        size_t off = 0;
        auto take = [&](size_t b) { size_t at = off; off += RoundUp<size_t>(b ? b : 1, 512); return at; };
        l.src2sorted = take(rows * 4);
        l.sorted2src = take(rows * 4);
        l.routing = take(cmx_moe_routing_workspace_bytes(static_cast<uint32_t>(rows), experts));
        l.meta = take(cmx_mx_gmm_workspace_bytes(experts));
        l.aCodes = take(rows * t.k);
        l.aScales = take(rows * mxops::ScaleCols(t.k));
        l.total = off;
        return l;
    }
    size_t GetWorkspaceSize(const CocTilingParams& t) override
    {
        return Arithmetic() == kInt8 ? Int8WorkspaceLayout(t).total : WorkspaceLayout(t).total;
    }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::DISPATCH_GMM_DEQUANT_SWIGLU; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (!CheckMoeCocTilingParams(t) || t.topK > t.expertNum) {
            return false;
        }
        if (rankSize != 1 || t.epSize != 1) {
            std::cerr << "DispatchGmmDequantSwiglu: this build runs one device's share (rankSize 1)" << std::endl;
            return false;
        }
        if (Arithmetic() == kInt8) {
            if (t.k % 128 != 0 || t.n % 64 != 0) {
                std::cerr << "INT8 DispatchGmmDequantSwiglu requires K % 128 == 0 and N % 64 == 0" << std::endl;
                return false;
            }
            return true;
        }
        if (t.k % 32 != 0 || t.n % 64 != 0) {
            std::cerr << "MX DispatchGmmDequantSwiglu requires K % 32 == 0 and N % 64 == 0" << std::endl;
            return false;
        }
        return true;
    }

    static int Launch(void* stream, const KernelParams& p, uint8_t* ws, const CocTilingParams& t)
    {
        if (Arithmetic() == kInt8) return LaunchInt8(stream, p, ws, t);
        const Layout l = WorkspaceLayout(t);
        const uint32_t experts = t.expertNum / t.epSize;
        const uint32_t rows = t.m * t.topK;
        const uint32_t sk = static_cast<uint32_t>(mxops::ScaleCols(t.k));
        int32_t* src2sorted = reinterpret_cast<int32_t*>(ws + l.src2sorted);
        int32_t* counts = reinterpret_cast<int32_t*>(p.customPtrs[3]);
        int rc = cmx_moe_init_routing(reinterpret_cast<const int32_t*>(p.customPtrs[0]), t.m, t.topK, experts,
                                      reinterpret_cast<int32_t*>(ws + l.sorted2src), src2sorted, counts, ws + l.routing, stream);
        if (rc != CMX_OK) return rc;
        rc = cmx_quant_scatter(p.ptrA, t.k, src2sorted, ws + l.aCodes, t.k, ws + l.aScales, sk, t.m, t.k, t.topK, stream);
        if (rc != CMX_OK) return rc;
        return cmx_mx_gmm_swiglu_quant(ws + l.aCodes, t.k, ws + l.aScales, sk, p.ptrB, p.customPtrs[1], p.ptrC, t.n / 2,
                                       p.customPtrs[2], static_cast<uint32_t>(mxops::ScaleCols(t.n / 2)), nullptr, counts, experts, rows,
                                       t.n, t.k, ws + l.meta, stream);
    }
};

REGISTER_OPERATOR("DispatchGmmDequantSwiglu", DispatchGmmDequantSwigluOperator);

#endif  // DISPATCH_GMM_DEQUANT_SWIGLU_HOST_H
