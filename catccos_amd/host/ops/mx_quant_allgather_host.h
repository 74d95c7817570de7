// "MxQuantAllGather" on one GPU: MX-quantise a bf16 [M, N] matrix; with one rank the gather is the
// identity, so the output is this rank's rows.  Host contract (buffer order, file names, checks) follows
// examples/ascend950_mx_quant_allgather/mx_quant_allgather_host.h:7-140; the element format is a run-time
// choice here instead of a compile-time macro.
#ifndef MX_QUANT_ALLGATHER_HOST_H
#define MX_QUANT_ALLGATHER_HOST_H

#include "op_common.h"

class MxQuantAllGatherOperator : public CatccosOperator {
public:
    static constexpr uint32_t MX_BLOCK_SIZE = 32;

    // CMX_FMT_E4M3 (default) / CMX_FMT_E5M2 / CMX_FMT_E2M1 / CMX_FMT_E1M2 and CMX_ROUND_RNE / CMX_ROUND_LUT for all instances
    static int& ElementFormat() { static int fmt = CMX_FMT_E4M3; return fmt; }
    static int& RoundMode() { static int mode = CMX_ROUND_RNE; return mode; }
    static uint32_t PackRatio() { return ElementFormat() == CMX_FMT_E2M1 || ElementFormat() == CMX_FMT_E1M2 ? 2 : 1; }

    static bool CheckProblemShape(uint32_t rankSize, const CocTilingParams& t)
    {
        return rankSize > 0 && rankSize <= MAX_RANK_SIZE && t.m > 0 && t.n > 0 && t.n % MX_BLOCK_SIZE == 0;
    }

    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t inputBytes = CheckedBufferSize({t.m, t.n, sizeof(uint16_t)});
        const size_t outputBytes = CheckedBufferSize({t.m, t.n / PackRatio(), t.rankSize});
        const size_t scaleBytes = static_cast<size_t>(t.m) * (t.n / MX_BLOCK_SIZE) * t.rankSize;
        uint8_t* input = nullptr;
        if (dataFile.empty()) {
            // default input: every element = rank + 1 (bf16)
            const float v = static_cast<float>(rankId + 1);
            uint32_t bits;
            std::memcpy(&bits, &v, 4);
            std::vector<uint16_t> fill(static_cast<size_t>(t.m) * t.n, static_cast<uint16_t>(bits >> 16));
            input = mxops::DeviceBufferFromValues(fill.data(), inputBytes);
        } else {
            input = mxops::DeviceBufferFromFile(inputBytes, mxops::RankFile(dataFile, "input", rankId, true));
        }
        uint8_t* output = mxrt::DeviceAlloc(outputBytes);
        uint8_t* mxScale = mxrt::DeviceAlloc(scaleBytes);
        params.SetKernelParams(input, mxScale, output);      // A = input, B = scales, C = codes
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t outputBytes = CheckedBufferSize({t.m, t.n / PackRatio(), t.rankSize});
        const size_t scaleBytes = static_cast<size_t>(t.m) * (t.n / MX_BLOCK_SIZE) * t.rankSize;
        mxops::DeviceBufferToFile(params.ptrC, outputBytes, mxops::RankFile(dataFile, "output", rankId, true));
        mxops::DeviceBufferToFile(params.ptrB, scaleBytes, mxops::RankFile(dataFile, "mxscale", rankId, true));
    }

    size_t GetWorkspaceSize(const CocTilingParams&) override { return 0; }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::MX_QUANT_ALLGATHER; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (!CheckProblemShape(rankSize, t)) {
            return false;
        }
        // quantised rows + scales of one block must fit this rank's share of the symmetric staging buffer
        const int32_t perRank = SHMEM_BUFF_BYTES / static_cast<int32_t>(rankSize) / static_cast<int32_t>(MAX_BLOCK_COUNT);
        const size_t blockBytes = CheckedBufferSize({t.m, static_cast<size_t>(t.n) + t.n / MX_BLOCK_SIZE});
        return blockBytes < static_cast<size_t>(perRank);
    }

    // Launch: the file format has exactly n/32 scale bytes per row; a scale pitch of exactly that many columns
    // makes the library write unpadded scale rows (odd block counts such as n = 96 included).
    static int Launch(void* stream, const KernelParams& params, const CocTilingParams& t, uint32_t rankId)
    {
        const uint32_t scaleCols = t.n / MX_BLOCK_SIZE;
        const uint32_t codeCols = t.n / PackRatio();
        uint8_t* codes = params.ptrC + static_cast<size_t>(rankId) * t.m * codeCols;
        uint8_t* scales = params.ptrB + static_cast<size_t>(rankId) * t.m * scaleCols;
        return cmx_mx_quant(params.ptrA, t.n, codes, codeCols, scales, scaleCols, t.m, t.n, ElementFormat(), RoundMode(),
                            stream);
    }
};

REGISTER_OPERATOR("MxQuantAllGather", MxQuantAllGatherOperator);

#endif  // MX_QUANT_ALLGATHER_HOST_H
