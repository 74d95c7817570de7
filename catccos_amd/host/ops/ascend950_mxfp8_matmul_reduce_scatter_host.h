// "Ascend950MxFp8MatmulReduceScatter" on one GPU: the device's full M x N x K MXFP8 product in bf16 (with
// one rank the reduce-scatter is the identity).  Host contract follows
// examples/ascend950_mxfp8_matmul_reduce_scatter/ascend950_mxfp8_matmul_reduce_scatter_host.h:28-147.
// Operand files come in either orientation, as the reference's generator writes them (scripts/
// gen_data_mxfp8_mmrs.py:309-330): A [M, K] with scales [M, K/64, 2], or [K, M] with [K/64, M, 2] when
// transA = 1; B [N, K] with [N, K/64, 2] when transB = 1 (the example's own setting), or [K, N] with
// [K/64, N, 2] when transB = 0.  Operands that are not K-contiguous are rewritten in the workspace first.
#ifndef ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER_HOST_H
#define ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER_HOST_H

#include "op_common.h"

class Ascend950MxFp8MatmulReduceScatterOperator : public CatccosOperator {
public:
    static int& ElementFormat() { static int fmt = CMX_FMT_E4M3; return fmt; }   // or CMX_FMT_E5M2

    static size_t ScaleRowBytes(uint32_t k) { return static_cast<size_t>(CeilDiv<size_t>(k, 64)) * 2; }

    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t aBytes = static_cast<size_t>(t.m) * t.k;
        const size_t bBytes = static_cast<size_t>(t.k) * t.n;
        const size_t cBytes = static_cast<size_t>(t.m) * t.n / t.rankSize * sizeof(uint16_t);
        const size_t aScaleBytes = static_cast<size_t>(t.m) * ScaleRowBytes(t.k);
        const size_t bScaleBytes = static_cast<size_t>(t.n) * ScaleRowBytes(t.k);
        auto file = [&](const char* stem) { return dataFile.empty() ? std::string() : mxops::RankFile(dataFile, stem, rankId, true); };
        // defaults without files: every code 60 (0x3C = 1.5), every scale byte 121 (2^-6)
        uint8_t* a = mxops::DeviceBufferFromFile(aBytes, file("a"), 60);
        uint8_t* b = mxops::DeviceBufferFromFile(bBytes, file("b"), 60);
        uint8_t* c = mxrt::DeviceAlloc(cBytes);
        uint8_t* aScale = mxops::DeviceBufferFromFile(aScaleBytes, file("a_scale"), 121);
        uint8_t* bScale = mxops::DeviceBufferFromFile(bScaleBytes, file("b_scale"), 121);
        params.SetKernelParams(a, b, c, aScale, bScale);
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t cBytes = static_cast<size_t>(t.m) * t.n / t.rankSize * sizeof(uint16_t);
        mxops::DeviceBufferToFile(params.ptrC, cBytes, dataFile + "/output.bin", rankId * cBytes);   // rank r at byte r*size
    }

    size_t GetWorkspaceSize(const CocTilingParams& t) override
    {
        return cmx_mx_gemm_ex_workspace_bytes(t.m, t.n, t.k, static_cast<int>(t.transA), static_cast<int>(t.transB));
    }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (rankSize != 1) {
            std::cerr << "Ascend950MxFp8MatmulReduceScatter: this build computes one device's product (rankSize 1)" << std::endl;
            return false;
        }
        if (t.transA > 1 || t.transB > 1) {
            std::cerr << "Ascend950MxFp8MatmulReduceScatter: transA and transB are 0 or 1" << std::endl;
            return false;
        }
        return t.k % 64 == 0;
    }

    static int Launch(void* stream, const KernelParams& params, uint8_t* workspace, const CocTilingParams& t)
    {
        return cmx_mx_gemm_ex(params.ptrA, params.customPtrs[0], params.ptrB, params.customPtrs[1], params.ptrC, t.n, t.m, t.n,
                              t.k, ElementFormat(), CMX_OUT_BF16, static_cast<int>(t.transA), static_cast<int>(t.transB),
                              workspace, stream);
    }
};

REGISTER_OPERATOR("Ascend950MxFp8MatmulReduceScatter", Ascend950MxFp8MatmulReduceScatterOperator);

#endif  // ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER_HOST_H
