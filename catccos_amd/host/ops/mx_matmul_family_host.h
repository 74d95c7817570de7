// The remaining MX matmul operators of the reference, on one GPU.  With one rank their collectives are the identity,
// so each of them is the device's own dense or grouped MX matmul behind that operator's name, buffer order and .bin
// file names:
//
//   Ascend950Fp8MxAllGatherMatmul         examples/ascend950_fp8_mx_allgather_matmul/..._host.h:20-133          dense   FP8
//   Ascend950Fp4MxAllGatherMatmul         examples/ascend950_fp4_mx_allgather_matmul/..._host.h                 dense   FP4
//   Ascend950MxFp8MatmulAllToAll          examples/ascend950_mxfp8_matmul_alltoall/..._host.h:28-125            dense   FP8
//   Ascend950Fp4MxMatmulReduceScatter     examples/ascend950_fp4_mx_matmul_reduce_scatter/..._host.h:20-110     dense   FP4
//   Ascend950MxFp8AllToAllMatmulSplitKUrma examples/ascend950_mxfp8_alltoall_matmul_split_k_urma/..._host.h:30-125 dense  FP8
//                                         (K is split over the ranks there: with one rank fullK = k, chunkM = m)
//   Ascend950Fp8MxAllToAllVGroupedMatmul  examples/ascend950_fp8_mx_alltoallv_grouped_matmul/..._host.h         grouped FP8
//   Ascend950Fp8MxGroupedMatmulAllToAllV  examples/ascend950_fp8_mx_grouped_matmul_alltoallv/..._host.h:18-180  grouped FP8
//   Ascend950Fp4MxGroupedMatmulAllToAllV  examples/ascend950_fp4_mx_grouped_matmul_alltoallv/..._host.h         grouped FP4
//
// All of them: A = codes [m, k], B = codes [k, n] per expert (transB = 0, their run scripts' setting) or [n, k]
// (transB = 1), C = fp16, custom = { A scales, B scales [, local tokens per expert, global tokens per local expert] }.
#ifndef MX_MATMUL_FAMILY_HOST_H
#define MX_MATMUL_FAMILY_HOST_H

#include "op_common.h"

namespace mxops {

enum class FileNames {
    kInputA,    // input_a_<r>.bin, input_b_<r>.bin, input_a_scale_<r>.bin, input_b_scale_<r>.bin
    kRankA,     // rank_<r>_a.bin, rank_<r>_b.bin, rank_<r>_a_scale.bin, rank_<r>_b_scale.bin
    kAGm,       // a_gm_<r>.bin, b_gm_<r>.bin, a_scale_<r>.bin, b_scale_<r>.bin
};

enum class OutputFile {
    kPerRank,   // output_<r>.bin
    kShared,    // output.bin, rank r at byte r * size
};

template <CocCommType kType, bool kFp4, bool kGrouped, FileNames kNames, OutputFile kOut>
class MxMatmulFamilyOperator : public CatccosOperator {
public:
    // FP8 operators: CMX_FMT_E4M3 (the examples' element type) or CMX_FMT_E5M2, for all instances
    static int& Fp8Format() { static int fmt = CMX_FMT_E4M3; return fmt; }
    static int Format() { return kFp4 ? CMX_FMT_E2M1 : Fp8Format(); }

    static std::string File(const std::string& dir, const char* what, uint32_t rankId)
    {
        const std::string r = std::to_string(rankId), w = what;
        switch (kNames) {
            case FileNames::kInputA: return dir + "/input_" + w + "_" + r + ".bin";
            case FileNames::kRankA: return dir + "/rank_" + r + "_" + w + ".bin";
            default: return dir + "/" + (w == "a" || w == "b" ? w + "_gm" : w) + "_" + r + ".bin";
        }
    }

    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t experts = kGrouped ? t.expertNum / t.epSize : 1;
        const size_t pack = kFp4 ? 2 : 1;
        const size_t scaleK = RoundUp<size_t>(CeilDiv<size_t>(t.k, 32), 2);
        const size_t aBytes = static_cast<size_t>(t.m) * t.k / pack;
        const size_t bBytes = static_cast<size_t>(t.k) * t.n * experts / pack;
        const size_t cBytes = static_cast<size_t>(t.m) * t.rankSize * t.n * sizeof(uint16_t);
        const bool fromFiles = !dataFile.empty();
        auto file = [&](const char* what) { return fromFiles ? File(dataFile, what, rankId) : std::string(); };
        // defaults without files: FP8 code 0x38 (1.0) / FP4 byte 0x22 (1.0, 1.0), scale byte 127 (2^0)
        uint8_t* a = DeviceBufferFromFile(aBytes, file("a"), kFp4 ? 0x22 : 0x38);
        uint8_t* b = DeviceBufferFromFile(bBytes, file("b"), kFp4 ? 0x22 : 0x38);
        uint8_t* aScale = DeviceBufferFromFile(static_cast<size_t>(t.m) * scaleK, file("a_scale"), 127);
        uint8_t* bScale = DeviceBufferFromFile(scaleK * t.n * experts, file("b_scale"), 127);
        uint8_t* c = DeviceBufferFromFile(cBytes, "", 0);          // rows past the routed ones stay zero, as the padded golden
        if (!kGrouped) {
            params.SetKernelParams(a, b, c, aScale, bScale);
            return;
        }
        const size_t localBytes = static_cast<size_t>(t.expertNum) * sizeof(int32_t);
        const size_t globalBytes = static_cast<size_t>(t.rankSize) * experts * sizeof(int32_t);
        uint8_t* local = nullptr;
        uint8_t* global = nullptr;
        if (fromFiles) {
            local = DeviceBufferFromFile(localBytes, dataFile + "/local_tokens_per_expert_" + std::to_string(rankId) + ".bin");
            global = DeviceBufferFromFile(globalBytes, dataFile + "/global_tokens_per_local_expert_" + std::to_string(rankId) + ".bin");
        } else {
            std::vector<int32_t> even(t.expertNum, static_cast<int32_t>(t.m / t.expertNum));
            local = DeviceBufferFromValues(even.data(), localBytes);
            global = DeviceBufferFromValues(even.data(), globalBytes);
        }
        params.SetKernelParams(a, b, c, aScale, bScale, local, global);
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t cBytes = static_cast<size_t>(t.m) * t.rankSize * t.n * sizeof(uint16_t);
        if (kOut == OutputFile::kShared) {
            DeviceBufferToFile(params.ptrC, cBytes, dataFile + "/output.bin", rankId * cBytes);
        } else {
            DeviceBufferToFile(params.ptrC, cBytes, dataFile + "/output_" + std::to_string(rankId) + ".bin");
        }
    }

    size_t GetWorkspaceSize(const CocTilingParams& t) override
    {
        if (kGrouped) return cmx_mx_gmm_ex_workspace_bytes(t.expertNum / (t.epSize ? t.epSize : 1), t.n, t.k, static_cast<int>(t.transB));
        return cmx_mx_gemm_ex_workspace_bytes(t.m, t.n, t.k, static_cast<int>(t.transA), static_cast<int>(t.transB));
    }
    CocCommType GetActualKernelType(const CocTilingParams&) override { return kType; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (kGrouped && !CheckMoeCocTilingParams(t)) return false;
        if (rankSize != 1 || (kGrouped && t.epSize != 1)) {
            std::cerr << CommTypeOpNameMap.at(kType) << ": this build computes one device's share (rankSize 1)" << std::endl;
            return false;
        }
        if (t.transA > 1 || t.transB > 1 || (kGrouped && t.transA != 0) || t.k % 64 != 0 || (kFp4 && t.n % 2 != 0)) {
            std::cerr << CommTypeOpNameMap.at(kType) << ": needs K % 64 == 0, transA / transB in {0, 1} (grouped: row-major A), even N for FP4"
                      << std::endl;
            return false;
        }
        return true;
    }

    static int Launch(void* stream, const KernelParams& p, uint8_t* workspace, const CocTilingParams& t)
    {
        if (kGrouped) {
            const uint32_t experts = t.expertNum / t.epSize;
            return cmx_mx_gmm_ex(p.ptrA, p.customPtrs[0], p.ptrB, p.customPtrs[1], p.ptrC, t.n,
                                 reinterpret_cast<const int32_t*>(p.customPtrs[3]), experts, t.m * t.rankSize, t.n, t.k, Format(),
                                 CMX_OUT_FP16, static_cast<int>(t.transB), workspace, stream);
        }
        return cmx_mx_gemm_ex(p.ptrA, p.customPtrs[0], p.ptrB, p.customPtrs[1], p.ptrC, t.n, t.m, t.n, t.k, Format(), CMX_OUT_FP16,
                              static_cast<int>(t.transA), static_cast<int>(t.transB), workspace, stream);
    }
};

}  // namespace mxops

class Ascend950Fp8MxAllGatherMatmulOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP8_MX_ALLGATHER_MATMUL, false, false, mxops::FileNames::kInputA, mxops::OutputFile::kPerRank> {};
class Ascend950Fp4MxAllGatherMatmulOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP4_MX_ALLGATHER_MATMUL, true, false, mxops::FileNames::kInputA, mxops::OutputFile::kPerRank> {};
class Ascend950MxFp8MatmulAllToAllOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_MXFP8_MATMUL_ALLTOALL, false, false, mxops::FileNames::kRankA, mxops::OutputFile::kPerRank> {};
class Ascend950MxFp8AllToAllMatmulSplitKUrmaOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA, false, false, mxops::FileNames::kInputA, mxops::OutputFile::kPerRank> {};
class Ascend950Fp4MxMatmulReduceScatterOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER, true, false, mxops::FileNames::kRankA, mxops::OutputFile::kShared> {};
class Ascend950Fp8MxAllToAllVGroupedMatmulOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, false, true, mxops::FileNames::kInputA, mxops::OutputFile::kPerRank> {};
class Ascend950Fp8MxGroupedMatmulAllToAllVOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, false, true, mxops::FileNames::kAGm, mxops::OutputFile::kPerRank> {};
class Ascend950Fp4MxGroupedMatmulAllToAllVOperator : public mxops::MxMatmulFamilyOperator<ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, true, true, mxops::FileNames::kAGm, mxops::OutputFile::kPerRank> {};

REGISTER_OPERATOR("Ascend950Fp8MxAllGatherMatmul", Ascend950Fp8MxAllGatherMatmulOperator);
REGISTER_OPERATOR("Ascend950Fp4MxAllGatherMatmul", Ascend950Fp4MxAllGatherMatmulOperator);
REGISTER_OPERATOR("Ascend950MxFp8MatmulAllToAll", Ascend950MxFp8MatmulAllToAllOperator);
REGISTER_OPERATOR("Ascend950MxFp8AllToAllMatmulSplitKUrma", Ascend950MxFp8AllToAllMatmulSplitKUrmaOperator);
REGISTER_OPERATOR("Ascend950Fp4MxMatmulReduceScatter", Ascend950Fp4MxMatmulReduceScatterOperator);
REGISTER_OPERATOR("Ascend950Fp8MxAllToAllVGroupedMatmul", Ascend950Fp8MxAllToAllVGroupedMatmulOperator);
REGISTER_OPERATOR("Ascend950Fp8MxGroupedMatmulAllToAllV", Ascend950Fp8MxGroupedMatmulAllToAllVOperator);
REGISTER_OPERATOR("Ascend950Fp4MxGroupedMatmulAllToAllV", Ascend950Fp4MxGroupedMatmulAllToAllVOperator);

#endif  // MX_MATMUL_FAMILY_HOST_H
