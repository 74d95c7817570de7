// Tiling arguments, buffer bundle and operator identifiers of the plugin surface.
// Same names, field order and enumerator values as the reference's utils/info.h:22-323, so a driver
// written against that header compiles against this one; the device runtime behind it is the
// cmx_rt_* shim instead of ACL.
#ifndef INFO_H
#define INFO_H

#include <climits>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <map>
#include <string>

#include "utils.h"

// ---- size constants (utils/info.h:22-43) -------------------------------------------------------
static uint64_t SHMEM_MALLOC_MAX_SIZE = 1024UL * 1024UL * 1024;
constexpr uint32_t M0 = 128;
constexpr uint32_t N0 = 256;
constexpr uint32_t K0 = 256;
constexpr uint32_t TILE_SHAPE_64 = 64;
constexpr uint32_t TILE_SHAPE_128 = 128;
constexpr uint32_t TILE_SHAPE_256 = 256;
constexpr uint32_t TILE_SHAPE_512 = 512;
constexpr uint32_t WORKSPACE_STAGES = 2;
constexpr uint32_t UB_STAGES = 2;
constexpr uint32_t BLOCK_NUM = 20;
constexpr uint32_t WARM_UP_TIMES = 10;
constexpr uint32_t PERF_TEST_CYCLE_TIMES = 3;
constexpr uint32_t MAX_BLOCK_COUNT = 2;
constexpr int32_t SHMEM_BUFF_BYTES = 1004UL * 1024 * 1024;
constexpr uint32_t IPC_BUFF_MAX_SIZE = 1000UL * 1024 * 1024;
constexpr uint32_t IPC_DATA_OFFSET = 2 * 1024 * 1024;
constexpr uint32_t PING_PONG_SIZE = 2;
constexpr uint32_t SYNC_UNIT_SIZE = 4 * sizeof(int64_t);
constexpr int32_t FLAG_BUFF_BYTES = 5 * 512 * 1024;
constexpr int32_t INPUT_DTYPE = 2;
constexpr int32_t MAX_RANK_SIZE = 128;

// ---- operator identifiers ------------------------------------------------------------------------
// One table drives the enum, the short-name lookup (utils/info.h:217-260) and the registry-name lookup
// (utils/info.h:271-313).  Row order fixes the enumerator values (utils/info.h:45-93); "" = no such name.
#define COC_COMM_TYPE_TABLE(X)                                                                                        \
    X(MATMUL_ALLREDUCE, "mmar", "MatmulAllReduce")                                                                    \
    X(ALLGATHER_MATMUL, "agmm", "AllGatherMatmul")                                                                    \
    X(ASCEND950_ALLGATHER_MATMUL, "a5agmm", "Ascend950AllGatherMatmul")                                               \
    X(MATMUL_REDUCE_SCATTER, "mmrs", "MatmulReduceScatter")                                                           \
    X(ASCEND950_MATMUL_REDUCE_SCATTER, "a5mmrs", "Ascend950MatmulReduceScatter")                                      \
    X(ALLGATHER_MATMUL_WITH_GATHER_RESULT, "agmmwg", "AllGatherMatmulWithGatherResult")                               \
    X(GROUPED_MATMUL_ALLTOALLV, "gmmata", "GroupedMatmulAllToAllV")                                                   \
    X(GROUPED_MATMUL_ALLTOALLV_TLA, "gmmatatla", "GroupedMatmulAllToAllVTla")                                         \
    X(ASCEND950_GROUPED_MATMUL_ALLTOALLV, "a5gmmata", "Ascend950GroupedMatmulAllToAllV")                              \
    X(ALLTOALLV_GROUPED_MATMUL, "atavgmm", "AllToAllVGroupedMatmul")                                                  \
    X(ALLGATHER_MATMUL_RDMA, "agmmrdma", "AllGatherMatmulRdma")                                                       \
    X(ALLTOALLV_GMM_V2, "atavgmmv2", "AllToAllVGMMV2")                                                                \
    X(ALLGATHER_MATMUL_DEQUANT_BIAS, "agmmdqbs", "AllGatherMatmulDequantBias")                                        \
    X(ALLGATHER_MATMUL_DEQUANT, "agmmdq", "AllGatherMatmulDequant")                                                   \
    X(ALLGATHER_MATMUL_DEQUANT_PADDING, "", "")                                                                       \
    X(QUANT_ALLTOALL, "", "")                                                                                         \
    X(QUANT_ALLGATHER, "", "")                                                                                        \
    X(MATMUL_DEQUANT_REDUCE_SCATTER_WRITE, "mmdqrs", "MatmulDequantReduceScatterWrite")                               \
    X(ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER, "a5mxfp8mmrs", "Ascend950MxFp8MatmulReduceScatter")                      \
    X(ASCEND950_MXFP8_MATMUL_ALLTOALL, "a5mxfp8mmata", "Ascend950MxFp8MatmulAllToAll")                                \
    X(ALLGATHER_MATMUL_REMOTE_READ, "agmmrr", "AllGatherMatmulRemoteRead")                                            \
    X(DISPATCH_GMM_DEQUANT_SWIGLU, "dgds", "DispatchGmmDequantSwiglu")                                                \
    X(ASCEND950_FP8_MX_ALLGATHER_MATMUL, "a5fp8mxagmm", "Ascend950Fp8MxAllGatherMatmul")                              \
    X(ASCEND950_FP4_MX_ALLGATHER_MATMUL, "a5fp4mxagmm", "Ascend950Fp4MxAllGatherMatmul")                              \
    X(MX_QUANT_ALLGATHER, "mxqtag", "MxQuantAllGather")                                                               \
    X(ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, "a5fp8gmmata", "Ascend950Fp8MxGroupedMatmulAllToAllV")               \
    X(ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, "a5fp4gmmata", "Ascend950Fp4MxGroupedMatmulAllToAllV")               \
    X(ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, "a5fp8mxatavgmm", "Ascend950Fp8MxAllToAllVGroupedMatmul")            \
    X(ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL, "a5fp4mxatavgmm", "Ascend950Fp4MxAllToAllVGroupedMatmul")            \
    X(ASCEND950_ALLTOALLV_GROUPED_MATMUL, "a5atavgmm", "Ascend950AllToAllVGroupedMatmul")                             \
    X(ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER, "a5fp4mmrs", "Ascend950Fp4MxMatmulReduceScatter")                       \
    X(DISPATCH_FFN_COMBINE, "moe", "DispatchFFNCombine")                                                              \
    X(ASCEND950_DISPATCH_FFN_COMBINE, "a5moe", "Ascend950DispatchFFNCombine")                                         \
    X(ASCEND950_ALLGATHER_MATMUL_UDMA, "a5agmmudma", "Ascend950AllGatherMatmulUdma")                                  \
    X(ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA, "a5mxfp8atammsplitkurma", "Ascend950MxFp8AllToAllMatmulSplitKUrma") \
    X(ASCEND950_MATMUL_REDUCE_SCATTER_UDMA, "a5mmrsudma", "Ascend950MatmulReduceScatterUdma")                         \
    X(ALLGATHER_MATMUL_SHALLOW_FUSION, "agmmsf", "AllGatherMatmulShallowFusion")                                      \
    X(MATMUL_ALLREDUCE_SHALLOW_FUSION, "mmarsf", "MatmulAllReduceShallowFusion")                                      \
    X(MATMUL_REDUCE_SCATTER_SHALLOW_FUSION, "mmrssf", "MatmulReduceScatterShallowFusion")                             \
    X(GROUPED_MATMUL_ALLTOALLV_SMALL_M, "gmmatasm", "GroupedMatmulAlltoAllvSmallM")                                   \
    X(ASCEND950_DISPATCH, "a5dispatch", "Ascend950Dispatch")                                                          \
    X(ASCEND950_MXFP8_ALLTOALL_MATMUL, "a5mxfp8atamm", "Ascend950MxFp8AllToAllMatmul")                                \
    X(ASCEND950_QUANT_MATMUL_ALLTOALL, "a5qmma", "Ascend950QuantMatmulAllToAll")                                      \
    X(ASCEND950_HIERARCHICAL_ALLTOALL, "", "")                                                                        \
    X(ASCEND950_BF16_ALLTOALL_MATMUL, "a5bf16atamm", "Ascend950Bf16AllToAllMatmul")

enum CocCommType {
#define COC_ENUM_ROW(id, shortName, opName) id,
    COC_COMM_TYPE_TABLE(COC_ENUM_ROW)
#undef COC_ENUM_ROW
    TYPE_NUM,
    UNKNOWN
};

enum CocDataType { FP16 = 1, INT8 = 2, BF16 = 27, FP8E4M3FN = 36 };

namespace coc_detail {
inline std::map<std::string, CocCommType> BuildShortNameMap()
{
    std::map<std::string, CocCommType> m;
#define COC_SHORT_ROW(id, shortName, opName) \
    if (shortName[0] != '\0') m.emplace(shortName, CocCommType::id);
    COC_COMM_TYPE_TABLE(COC_SHORT_ROW)
#undef COC_SHORT_ROW
    return m;
}
inline std::map<CocCommType, std::string> BuildOpNameMap()
{
    std::map<CocCommType, std::string> m;
#define COC_OP_ROW(id, shortName, opName) \
    if (opName[0] != '\0') m.emplace(CocCommType::id, opName);
    COC_COMM_TYPE_TABLE(COC_OP_ROW)
#undef COC_OP_ROW
    return m;
}
}  // namespace coc_detail

// short kernel name -> identifier, identifier -> registry name
const std::map<std::string, CocCommType> CommTypeMap = coc_detail::BuildShortNameMap();
const std::map<CocCommType, std::string> CommTypeOpNameMap = coc_detail::BuildOpNameMap();

inline CocCommType GetCommType(const std::string& kernelName)
{
    const auto it = CommTypeMap.find(kernelName);
    return it == CommTypeMap.end() ? CocCommType::UNKNOWN : it->second;
}

// ---- tiling arguments (utils/info.h:97-126) --------------------------------------------------------
// All uint32_t, passed by value to the launch.  m is tokens per rank before top-k expansion for the MoE
// operators; n is the GMM1 width (gate + up).
struct CocTilingParams {
    uint32_t m = 0;
    uint32_t k = 0;
    uint32_t n = 0;
    uint32_t transA = 0;
    uint32_t transB = 0;
    uint32_t m0 = 0;
    uint32_t k0 = 0;
    uint32_t n0 = 0;
    uint32_t commTileM = 0;
    uint32_t commInterval = 0;
    uint32_t commNpuSplit = 0;
    uint32_t commDataSplit = 0;
    uint32_t commBlockM = 0;
    uint32_t rankSize = 0;
    uint32_t epSize = 0;
    uint32_t expertNum = 0;
    uint32_t topK = 1;
};

inline bool CheckCommonCocTilingParams(uint32_t rankSize, const CocTilingParams& params)
{
    const bool ranksAgree = rankSize > 0 && params.rankSize == rankSize;
    const bool shapePositive = params.m > 0 && params.k > 0 && params.n > 0;
    const bool tilePositive = params.m0 > 0 && params.k0 > 0 && params.n0 > 0;
    return ranksAgree && shapePositive && tilePositive;
}

inline bool CheckMoeCocTilingParams(const CocTilingParams& params)
{
    if (params.epSize == 0 || params.expertNum == 0 || params.topK == 0) {
        return false;
    }
    return params.expertNum % params.epSize == 0;
}

struct COCMatMulInfo {
    int64_t m;
    int64_t k;
    int64_t n;
};

// ---- buffer bundle (utils/info.h:134-214) -----------------------------------------------------------
// ptrA/ptrB/ptrC plus an owned host array of extra device pointers.  Move-only: the array's lifetime is
// this object's.  The device buffers themselves belong to the caller (FreeDeviceSpace).
struct KernelParams {
    uint8_t* ptrA = nullptr;
    uint8_t* ptrB = nullptr;
    uint8_t* ptrC = nullptr;
    uint8_t** customPtrs = nullptr;
    uint32_t customCount = 0;

    KernelParams() = default;
    KernelParams(const KernelParams&) = delete;
    KernelParams& operator=(const KernelParams&) = delete;
    KernelParams& operator=(KernelParams&&) = delete;

    KernelParams(KernelParams&& other) noexcept
        : ptrA(other.ptrA), ptrB(other.ptrB), ptrC(other.ptrC), customPtrs(other.customPtrs),
          customCount(other.customCount)
    {
        other.ptrA = other.ptrB = other.ptrC = nullptr;
        other.customPtrs = nullptr;
        other.customCount = 0;
    }

    template <typename... Args>
    void SetKernelParams(uint8_t* a, uint8_t* b, uint8_t* c, Args... args)
    {
        ptrA = a;
        ptrB = b;
        ptrC = c;
        ReleaseCustom();
        constexpr uint32_t extra = sizeof...(args);
        customCount = extra;
        if constexpr (extra > 0) {
            customPtrs = static_cast<uint8_t**>(std::malloc(extra * sizeof(uint8_t*)));
            uint8_t* list[] = {args...};
            for (uint32_t i = 0; i < extra; ++i) {
                customPtrs[i] = list[i];
            }
        }
    }

    ~KernelParams() { ReleaseCustom(); }

private:
    void ReleaseCustom()
    {
        std::free(customPtrs);      // plain host memory: the array is only read by host code
        customPtrs = nullptr;
    }
};

// Frees every device buffer the bundle names (the operator's AllocateDeviceSpace allocated them).
inline void FreeDeviceSpace(KernelParams& params)
{
    for (uint8_t** slot : {&params.ptrA, &params.ptrB, &params.ptrC}) {
        if (*slot != nullptr) {
            MX_CHECK(cmx_rt_free(*slot));
            *slot = nullptr;
        }
    }
    for (uint32_t i = 0; i < params.customCount; ++i) {
        if (params.customPtrs[i] != nullptr) {
            MX_CHECK(cmx_rt_free(params.customPtrs[i]));
            params.customPtrs[i] = nullptr;
        }
    }
}

inline int32_t CeilDev(int32_t num, int32_t div)
{
    return div == 0 ? 0 : (num + div - 1) / div;
}

#endif  // INFO_H
