// "Ascend950Fp4MxAllToAllVGroupedMatmul" on one GPU: MXFP4 (E2M1 x2 per byte) grouped matmul over the
// rows of each local expert, fp16 output.  With one rank the all-to-all is the identity: A's rows already
// sit in expert order.  Host contract follows
// examples/ascend950_fp4_mx_alltoallv_grouped_matmul/ascend950_fp4_mx_alltoallv_grouped_matmul_host.h:16-184.
// B comes in either orientation of the reference's generator (examples/utils/gen_data_fp4_mx_alltoallv_gmm.py:586-620):
// [E, K, N/2] bytes with scales [E, K/64, N, 2] (transB = 0, the setting of the example's run.sh) or [E, N, K/2] with
// [E, N, K/64, 2] (transB = 1); the first is rewritten K-contiguous in the workspace before the matmul.
#ifndef ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL_HOST_H
#define ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL_HOST_H

#include "op_common.h"

class Ascend950Fp4MxAllToAllVGroupedMatmulOperator : public CatccosOperator {
public:
    // custom = { A scale [m, k/32], B scale [E, n, k/32], localTokensPerExpert i32 [expertNum],
    //            globalTokensPerLocalExpert i32 [rankSize, E] }
    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t experts = t.expertNum / t.epSize;
        const size_t scaleK = CeilDiv<size_t>(t.k, 32);
        const size_t aBytes = static_cast<size_t>(t.m) * t.k / 2;
        const size_t bBytes = static_cast<size_t>(t.k) * t.n * experts / 2;
        const size_t cBytes = static_cast<size_t>(t.m) * t.n * t.rankSize * sizeof(uint16_t);
        const size_t aScaleBytes = static_cast<size_t>(t.m) * scaleK;
        const size_t bScaleBytes = scaleK * t.n * experts;
        const size_t localBytes = static_cast<size_t>(t.expertNum) * sizeof(int32_t);
        const size_t globalBytes = static_cast<size_t>(t.rankSize) * experts * sizeof(int32_t);
        const bool fromFiles = !dataFile.empty();
        auto file = [&](const char* stem) { return fromFiles ? mxops::RankFile(dataFile, stem, rankId, false) : std::string(); };
        uint8_t* a = mxops::DeviceBufferFromFile(aBytes, file("input_a"), 1);
        uint8_t* b = mxops::DeviceBufferFromFile(bBytes, file("input_b"), 1);
        uint8_t* aScale = mxops::DeviceBufferFromFile(aScaleBytes, file("input_a_scale"), 1);
        uint8_t* bScale = mxops::DeviceBufferFromFile(bScaleBytes, file("input_b_scale"), 1);
        uint8_t* local = nullptr;
        uint8_t* global = nullptr;
        if (fromFiles) {
            local = mxops::DeviceBufferFromFile(localBytes, file("local_tokens_per_expert"));
            global = mxops::DeviceBufferFromFile(globalBytes, file("global_tokens_per_local_expert"));
        } else {
            std::vector<uint32_t> l(t.expertNum, t.m / t.expertNum);
            std::vector<uint32_t> g(t.rankSize * experts, t.m / t.expertNum * t.rankSize / t.epSize);
            local = mxops::DeviceBufferFromValues(l.data(), localBytes);
            global = mxops::DeviceBufferFromValues(g.data(), globalBytes);
        }
        uint8_t* c = mxrt::DeviceAlloc(cBytes);
        MX_CHECK(cmx_rt_memset(c, 0, cBytes));       // rows past the routed ones stay zero, as the padded golden
        params.SetKernelParams(a, b, c, aScale, bScale, local, global);
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t cBytes = static_cast<size_t>(t.m) * t.rankSize * t.n * sizeof(uint16_t);
        mxops::DeviceBufferToFile(params.ptrC, cBytes, mxops::RankFile(dataFile, "output", rankId, false));
    }

    size_t GetWorkspaceSize(const CocTilingParams& t) override
    {
        return cmx_mx_gmm_ex_workspace_bytes(t.expertNum / (t.epSize ? t.epSize : 1), t.n, t.k, static_cast<int>(t.transB));
    }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (!CheckMoeCocTilingParams(t)) {
            return false;
        }
        if (rankSize != 1 || t.epSize != 1) {
            std::cerr << "Ascend950Fp4MxAllToAllVGroupedMatmul: this build runs one device's share (rankSize 1)" << std::endl;
            return false;
        }
        const uint32_t kLoop = CeilDev(t.k, t.k0);
        const int64_t maxPeerMemPerRank = 2LL * IPC_BUFF_MAX_SIZE / rankSize / MAX_BLOCK_COUNT;
        if (static_cast<int64_t>(t.commInterval) * t.m0 * t.k0 * kLoop >= maxPeerMemPerRank) {
            return false;
        }
        if (t.transA != 0 || t.transB > 1 || t.k % 64 != 0 || (t.transB == 0 && t.n % 2 != 0)) {
            std::cerr << "MXFP4 grouped matmul needs row-major A, transB 0 or 1, K % 64 == 0 (and an even N with transB = 0)" << std::endl;
            return false;
        }
        return true;
    }

    static int Launch(void* stream, const KernelParams& p, uint8_t* workspace, const CocTilingParams& t)
    {
        const uint32_t experts = t.expertNum / t.epSize;
        return cmx_mx_gmm_ex(p.ptrA, p.customPtrs[0], p.ptrB, p.customPtrs[1], p.ptrC, t.n,
                             reinterpret_cast<const int32_t*>(p.customPtrs[3]), experts, t.m * t.rankSize, t.n, t.k, CMX_FMT_E2M1,
                             CMX_OUT_FP16, static_cast<int>(t.transB), workspace, stream);
    }
};

REGISTER_OPERATOR("Ascend950Fp4MxAllToAllVGroupedMatmul", Ascend950Fp4MxAllToAllVGroupedMatmulOperator);

#endif  // ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL_HOST_H
