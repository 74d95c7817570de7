// catccos_mx_run - single-GPU driver over the operator registry.
//
//   catccos_mx_run <operator> M K N [options]
//     <operator>    registry name ("Ascend950DispatchFFNCombine", ...) or short name ("a5moe", "mxqtag",
//                   "a5mxfp8mmrs", "a5fp4mxatavgmm", "dgds", "a5fp8mxagmm", "a5fp4mxagmm", "a5mxfp8mmata", "a5fp4mmrs",
//                   "a5fp8mxatavgmm", "a5fp8gmmata", "a5fp4gmmata")
//     --experts E   local experts (MoE operators; default 4)      --topk T     routes per token (default 4)
//     --data DIR    directory with the operator's input .bin files; outputs are written there too
//                   (without it inputs are defaults / zeros and nothing is written)
//     --fmt F       e4m3 | e5m2 | e2m1 | e1m2 for the quantizer, e4m3 | e5m2 for the dense matmul (default e4m3)
//     --arith A     mx | int8 for DispatchGmmDequantSwiglu (default mx; int8 = the reference operator's own arithmetic
//                   and file names: a_gm, b_gm, scale_gm, expert_idx -> output)
//     --transa 0|1  dense matmul: A files hold [K, M] / [K/64, M, 2] when 1 (default 0)
//     --transb 0|1  dense matmul: B files hold [K, N] / [K/64, N, 2] when 0 (default 1: [N, K])
//     --repeats R   launches per case (default 1)               --warmup W   untimed launches (default 5)
//     --poison      fill workspace and outputs with 0xA5 first (stale-state check)
//     --m0 128|256  recorded in the tiling arguments (GMM1 M tile of the reference; tile choice here is automatic)
//
// The flow is the reference examples': create by name -> ValidateCocTilingParams -> GetWorkspaceSize ->
// AllocateDeviceSpace -> launch -> synchronize -> WriteResultFile -> FreeDeviceSpace, with the same
// "[TEST]" / "[CONFIG]" log lines.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>

#include "launch_map.h"
#include "ops/ascend950_mxfp8_matmul_reduce_scatter_host.h"
#include "ops/dispatch_gmm_dequant_swiglu_host.h"
#include "ops/mx_matmul_family_host.h"
#include "ops/mx_quant_allgather_host.h"

namespace {

struct Options {
    std::string op;
    uint32_t m = 0, k = 0, n = 0, experts = 4, topK = 4, repeats = 1, warmup = 5, m0 = M0, transA = 0, transB = 1;
    std::string data, fmt = "e4m3", arith = "mx";
    bool poison = false;
};

uint32_t ParsePositive(const char* text, const char* name)
{
    char* end = nullptr;
    const unsigned long v = std::strtoul(text, &end, 10);
    if (end == text || *end != '\0' || v == 0 || v > 0xFFFFFFFFul) {
        throw std::runtime_error(std::string(name) + " must be a positive uint32 integer");
    }
    return static_cast<uint32_t>(v);
}

Options Parse(int argc, char** argv)
{
    if (argc < 5) {
        throw std::runtime_error("Usage: catccos_mx_run <operator> M K N [--experts E] [--topk T] [--data DIR] [--fmt F] "
                                 "[--repeats R] [--warmup W] [--poison] [--m0 128|256] [--transa 0|1] [--transb 0|1] [--arith mx|int8]");
    }
    Options o;
    o.op = argv[1];
    o.m = ParsePositive(argv[2], "M");
    o.k = ParsePositive(argv[3], "K");
    o.n = ParsePositive(argv[4], "N");
    for (int i = 5; i < argc; ++i) {
        const std::string a = argv[i];
        auto next = [&](const char* name) -> const char* {
            if (i + 1 >= argc) throw std::runtime_error(std::string(name) + " needs a value");
            return argv[++i];
        };
        if (a == "--experts") o.experts = ParsePositive(next("--experts"), "experts");
        else if (a == "--topk") o.topK = ParsePositive(next("--topk"), "topK");
        else if (a == "--repeats") o.repeats = ParsePositive(next("--repeats"), "repeats");
        else if (a == "--warmup") o.warmup = static_cast<uint32_t>(std::strtoul(next("--warmup"), nullptr, 10));
        else if (a == "--m0") o.m0 = ParsePositive(next("--m0"), "m0");
        else if (a == "--transa") o.transA = static_cast<uint32_t>(std::strtoul(next("--transa"), nullptr, 10));
        else if (a == "--transb") o.transB = static_cast<uint32_t>(std::strtoul(next("--transb"), nullptr, 10));
        else if (a == "--data") o.data = next("--data");
        else if (a == "--fmt") o.fmt = next("--fmt");
        else if (a == "--arith") o.arith = next("--arith");
        else if (a == "--poison") o.poison = true;
        else throw std::runtime_error("unknown option " + a);
    }
    if (o.m0 != 128 && o.m0 != 256) throw std::runtime_error("Invalid GMM1 M tile");
    if (o.arith != "mx" && o.arith != "int8") throw std::runtime_error("unknown arithmetic " + o.arith);
    return o;
}

int FormatOf(const std::string& f)
{
    if (f == "e4m3") return CMX_FMT_E4M3;
    if (f == "e5m2") return CMX_FMT_E5M2;
    if (f == "e2m1") return CMX_FMT_E2M1;
    if (f == "e1m2") return CMX_FMT_E1M2;
    throw std::runtime_error("unknown element format " + f);
}

int Run(int argc, char** argv)
{
    const Options o = Parse(argc, argv);
    CocCommType type = GetCommType(o.op);
    std::string opName = o.op;
    if (type != CocCommType::UNKNOWN) {
        opName = CommTypeOpNameMap.at(type);
    } else {
        for (const auto& kv : CommTypeOpNameMap) {
            if (kv.second == o.op) type = kv.first;
        }
    }
    auto op = OperatorRegistry::Instance().CreateOperator(opName);
    if (!op) {
        std::cout << "Operator " << opName << " not found!" << std::endl;
        return -1;
    }
    const int fmt = FormatOf(o.fmt);
    MxQuantAllGatherOperator::ElementFormat() = fmt;
    DispatchGmmDequantSwigluOperator::Arithmetic() =
        o.arith == "int8" ? DispatchGmmDequantSwigluOperator::kInt8 : DispatchGmmDequantSwigluOperator::kMx;
    if (fmt == CMX_FMT_E4M3 || fmt == CMX_FMT_E5M2) {
        Ascend950Fp8MxAllGatherMatmulOperator::Fp8Format() = fmt;
        Ascend950MxFp8MatmulAllToAllOperator::Fp8Format() = fmt;
        Ascend950MxFp8AllToAllMatmulSplitKUrmaOperator::Fp8Format() = fmt;
        Ascend950Fp8MxAllToAllVGroupedMatmulOperator::Fp8Format() = fmt;
        Ascend950Fp8MxGroupedMatmulAllToAllVOperator::Fp8Format() = fmt;
    }
    const bool fp4 = fmt == CMX_FMT_E2M1 || fmt == CMX_FMT_E1M2;
    MxQuantAllGatherOperator::RoundMode() = fp4 ? CMX_ROUND_LUT : CMX_ROUND_RNE;
    Ascend950MxFp8MatmulReduceScatterOperator::ElementFormat() = fp4 ? CMX_FMT_E4M3 : fmt;

    const uint32_t rankSize = 1, rankId = 0;
    CocTilingParams tiling{};
    tiling.m = o.m;
    tiling.k = o.k;
    tiling.n = o.n;
    tiling.transA = o.transA;
    tiling.transB = o.transB;
    tiling.m0 = o.m0;
    tiling.n0 = N0;
    tiling.k0 = K0;
    tiling.commTileM = 64;
    tiling.commInterval = 10;
    tiling.commNpuSplit = rankSize;
    tiling.commDataSplit = 1;
    tiling.commBlockM = 64;
    tiling.rankSize = rankSize;
    tiling.epSize = rankSize;
    tiling.expertNum = rankSize * o.experts;
    tiling.topK = o.topK;

    std::cout << "[TEST] input rank_size: " << rankSize << " rank_id:" << rankId << " operator: " << opName << std::endl;
    if (!op->ValidateCocTilingParams(rankSize, tiling)) {
        std::cerr << "Invalid CocTilingParams" << std::endl;
        return -1;
    }
    // the operators with fp16 output are registered under FP16, the others under BF16
    KernelFuncPtr launch = GetKernelFunc(op->GetActualKernelType(tiling), BF16);
    if (!launch) launch = GetKernelFunc(op->GetActualKernelType(tiling), FP16);
    if (!launch) {
        std::cerr << "[ERROR] no launch entry for " << opName << std::endl;
        return 1;
    }
    int devices = 0;
    MxCheckOrThrow(cmx_rt_device_count(&devices), "device count");
    if (devices < 1) throw std::runtime_error("no GPU visible");
    MxCheckOrThrow(cmx_rt_set_device(0), "set device");
    cmx_stream_t stream = nullptr;
    MxCheckOrThrow(cmx_rt_stream_create(&stream), "stream create");

    const size_t workspaceSize = op->GetWorkspaceSize(tiling);
    std::cout << "[CONFIG] M=" << o.m << " K=" << o.k << " N=" << o.n << " experts=" << o.experts << " topK=" << o.topK
              << " fmt=" << o.fmt << " workspace_bytes=" << workspaceSize << " symmetric_bytes=" << op->GetSymmetricSize(tiling)
              << " (unused with one rank)" << std::endl;
    KernelParams params;
    op->AllocateDeviceSpace(params, tiling, rankId, o.data);
    uint8_t* workspace = workspaceSize ? mxrt::DeviceAlloc(workspaceSize) : nullptr;
    if (o.poison && workspace) MxCheckOrThrow(cmx_rt_memset(workspace, 0xA5, workspaceSize), "poison");

    auto once = [&]() {
        launch(stream, 0, 0, params, workspace, nullptr, tiling, tiling.transA, tiling.transB);
        MxCheckOrThrow(LaunchStatus(), "launch");
    };
    for (uint32_t i = 0; i < o.warmup; ++i) once();
    MxCheckOrThrow(cmx_rt_stream_sync(stream), "synchronize");
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t i = 0; i < o.repeats; ++i) once();
    MxCheckOrThrow(cmx_rt_stream_sync(stream), "synchronize");
    const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / o.repeats;
    std::cout << "[TEST] " << opName << " avg " << us << " us over " << o.repeats << " launches" << std::endl;

    if (!o.data.empty()) {
        op->WriteResultFile(params, tiling, rankId, o.data);
    }
    FreeDeviceSpace(params);
    if (workspace) MX_CHECK(cmx_rt_free(workspace));
    MX_CHECK(cmx_rt_stream_destroy(stream));
    std::cout << "[TEST] begin to exit...... rankId: " << rankId << std::endl;
    return 0;
}

}  // namespace

int main(int argc, char** argv)
{
    try {
        return Run(argc, argv);
    } catch (const std::exception& error) {
        std::cerr << "[ERROR] " << error.what() << std::endl;
        return 1;
    }
}
