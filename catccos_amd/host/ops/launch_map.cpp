// Launch table of the operators this build implements (see include/launch_map.h).
#include "launch_map.h"

#include "ascend950_dispatch_ffn_combine_host.h"
#include "ascend950_fp4_mx_alltoallv_grouped_matmul_host.h"
#include "ascend950_mxfp8_matmul_reduce_scatter_host.h"
#include "dispatch_gmm_dequant_swiglu_host.h"
#include "mx_matmul_family_host.h"
#include "mx_quant_allgather_host.h"

namespace {

void LaunchQuant(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t*, uint8_t*, CocTilingParams& t, uint32_t, uint32_t)
{
    LaunchStatus() = MxQuantAllGatherOperator::Launch(stream, p, t, 0);
}
void LaunchMmrs(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t* ws, uint8_t*, CocTilingParams& t, uint32_t transA, uint32_t transB)
{
    CocTilingParams tt = t;
    tt.transA = transA;
    tt.transB = transB;
    LaunchStatus() = Ascend950MxFp8MatmulReduceScatterOperator::Launch(stream, p, ws, tt);
}
void LaunchFfn(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t* ws, uint8_t* symm, CocTilingParams& t, uint32_t, uint32_t)
{
    LaunchStatus() = Ascend950DispatchFFNCombineOperator::Launch(stream, p, p.ptrC, ws, symm, t);
}
void LaunchFp4Gmm(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t* ws, uint8_t*, CocTilingParams& t, uint32_t transA, uint32_t transB)
{
    CocTilingParams tt = t;
    tt.transA = transA;
    tt.transB = transB;
    LaunchStatus() = Ascend950Fp4MxAllToAllVGroupedMatmulOperator::Launch(stream, p, ws, tt);
}
void LaunchDgds(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t* ws, uint8_t*, CocTilingParams& t, uint32_t, uint32_t)
{
    LaunchStatus() = DispatchGmmDequantSwigluOperator::Launch(stream, p, ws, t);
}

template <class Op>
void LaunchFamily(void* stream, uint32_t, uint64_t, KernelParams& p, uint8_t* ws, uint8_t*, CocTilingParams& t, uint32_t transA, uint32_t transB)
{
    CocTilingParams tt = t;
    tt.transA = transA;
    tt.transB = transB;
    LaunchStatus() = Op::Launch(stream, p, ws, tt);
}

}  // namespace

std::map<uint32_t, KernelFuncPtr>& LaunchMap()
{
    static std::map<uint32_t, KernelFuncPtr> table = {
        {LaunchKey(MX_QUANT_ALLGATHER, BF16), LaunchQuant},
        {LaunchKey(ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER, BF16), LaunchMmrs},
        {LaunchKey(ASCEND950_MXFP8_MATMUL_REDUCE_SCATTER, FP8E4M3FN), LaunchMmrs},
        {LaunchKey(ASCEND950_DISPATCH_FFN_COMBINE, BF16), LaunchFfn},
        {LaunchKey(ASCEND950_FP4_MX_ALLTOALLV_GROUPED_MATMUL, FP16), LaunchFp4Gmm},
        {LaunchKey(DISPATCH_GMM_DEQUANT_SWIGLU, BF16), LaunchDgds},
        {LaunchKey(ASCEND950_FP8_MX_ALLGATHER_MATMUL, FP16), LaunchFamily<Ascend950Fp8MxAllGatherMatmulOperator>},
        {LaunchKey(ASCEND950_FP4_MX_ALLGATHER_MATMUL, FP16), LaunchFamily<Ascend950Fp4MxAllGatherMatmulOperator>},
        {LaunchKey(ASCEND950_MXFP8_MATMUL_ALLTOALL, FP16), LaunchFamily<Ascend950MxFp8MatmulAllToAllOperator>},
        {LaunchKey(ASCEND950_MXFP8_ALLTOALL_MATMUL_SPLIT_K_URMA, FP16), LaunchFamily<Ascend950MxFp8AllToAllMatmulSplitKUrmaOperator>},
        {LaunchKey(ASCEND950_FP4_MX_MATMUL_REDUCE_SCATTER, FP16), LaunchFamily<Ascend950Fp4MxMatmulReduceScatterOperator>},
        {LaunchKey(ASCEND950_FP8_MX_ALLTOALLV_GROUPED_MATMUL, FP16), LaunchFamily<Ascend950Fp8MxAllToAllVGroupedMatmulOperator>},
        {LaunchKey(ASCEND950_FP8_MX_GROUPED_MATMUL_ALLTOALLV, FP16), LaunchFamily<Ascend950Fp8MxGroupedMatmulAllToAllVOperator>},
        {LaunchKey(ASCEND950_FP4_MX_GROUPED_MATMUL_ALLTOALLV, FP16), LaunchFamily<Ascend950Fp4MxGroupedMatmulAllToAllVOperator>},
    };
    return table;
}

KernelFuncPtr GetKernelFunc(CocCommType type, CocDataType dtype)
{
    auto& table = LaunchMap();
    const auto it = table.find(LaunchKey(type, dtype));
    return it == table.end() ? nullptr : it->second;
}
