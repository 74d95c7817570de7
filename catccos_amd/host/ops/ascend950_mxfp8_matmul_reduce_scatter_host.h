// "Ascend950MxFp8MatmulReduceScatter" on one GPU: the device's full M x N x K MXFP8 product in bf16 (with
// one rank the reduce-scatter is the identity).  Host contract follows
// examples/ascend950_mxfp8_matmul_reduce_scatter/ascend950_mxfp8_matmul_reduce_scatter_host.h:28-147.
// B must be stored transposed ([N, K] codes, [N, K/64, 2] scales; transB = 1): both operands K-contiguous.
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

    size_t GetWorkspaceSize(const CocTilingParams&) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (rankSize != 1) {
            std::cerr << "Ascend950MxFp8MatmulReduceScatter: this build computes one device's product (rankSize 1)" << std::endl;
            return false;
        }
        if (t.transA != 0 || t.transB != 1) {
            std::cerr << "Ascend950MxFp8MatmulReduceScatter: A row-major and B transposed ([N,K]) are required" << std::endl;
            return false;
        }
        return t.k % 64 == 0;
    }

    static int Launch(void* stream, const KernelParams& params, const CocTilingParams& t)
    {
        const uint32_t ldScale = static_cast<uint32_t>(ScaleRowBytes(t.k));
        return cmx_mx_gemm(params.ptrA, t.k, params.customPtrs[0], ldScale, params.ptrB, t.k, params.customPtrs[1], ldScale,
                           params.ptrC, t.n, t.m, t.n, t.k, ElementFormat(), CMX_OUT_BF16, stream);
    }
};

REGISTER_OPERATOR("Ascend950MxFp8MatmulReduceScatter", Ascend950MxFp8MatmulReduceScatterOperator);

#endif  // ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER_HOST_H
