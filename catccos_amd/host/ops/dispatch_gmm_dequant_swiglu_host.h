// "DispatchGmmDequantSwiglu" in MXFP8 on one GPU: route tokens to experts, quantise + scatter them,
// grouped matmul with the gate|up weights, dequant, SwiGLU, and MX requant of the result.
// The reference operator of this name (examples/dispatch_gmm_dequant_swiglu/dispatch_gmm_dequant_swiglu_host.h)
// is an INT8 per-token/per-channel kernel; this class keeps its name, buffer roles and workspace contract
// and restates the arithmetic in MX (the chain examples/utils/gen_data_moe.py:628-658 up to the requant).
#ifndef DISPATCH_GMM_DEQUANT_SWIGLU_HOST_H
#define DISPATCH_GMM_DEQUANT_SWIGLU_HOST_H

#include "op_common.h"

class DispatchGmmDequantSwigluOperator : public CatccosOperator {
public:
    // ptrA = x bf16 [m,k], ptrB = W1 [E,n,k], ptrC = act codes E4M3 [m*topK, n/2],
    // custom = { expertIdx i32 [m,topK], W1 scale [E,n,k/32], act scales [m*topK, n/64], tokens per expert i32 [E] }
    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
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
    size_t GetWorkspaceSize(const CocTilingParams& t) override { return WorkspaceLayout(t).total; }
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
        if (t.k % 32 != 0 || t.n % 64 != 0) {
            std::cerr << "MX DispatchGmmDequantSwiglu requires K % 32 == 0 and N % 64 == 0" << std::endl;
            return false;
        }
        return true;
    }

    static int Launch(void* stream, const KernelParams& p, uint8_t* ws, const CocTilingParams& t)
    {
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
