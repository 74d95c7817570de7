// Host-only checks of the plugin surface (no GPU work): registry behaviour, tiling validation, sizing
// known answers of the reference's own host tests, and the raw-file helpers.
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <vector>

#include "catccos/detail/ascend950_moe_ub.h"
#include "launch_map.h"
#include "ops/ascend950_dispatch_ffn_combine_host.h"
#include "ops/mx_quant_allgather_host.h"

#define EXPECT(cond)                                                                     \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            std::cerr << "FAILED " << __FILE__ << ":" << __LINE__ << " " #cond << std::endl; \
            return EXIT_FAILURE;                                                         \
        }                                                                                \
    } while (0)

int main()
{
    using Ready = Catccos::Detail::Ascend950MoeReady;
    using Ub = Catccos::Detail::Ascend950MoeUb;
    // tests/ascend950/test_moe_ready_capacity.cpp:18-19 and test_moe_ub_capacity.cpp:19-38
    static_assert(Ready::SwigluRegionBytes(1024, 32) == 2048);
    static_assert(Ready::DispatchRegionBytes(1024, 2, 32) == 2560);
    static_assert(Ub::UnpermuteBytes(512, 2048, 8, 48) == 37760 && Ub::InputQuantBytes(2048) == 12928 && Ub::DispatchBytes(2048) == 8448);
    static_assert(Ub::UnpermuteBytes(1, 256, 1, 48) == 9536);
    EXPECT(Ub::Fits(1, 14336, 8, 48) && !Ub::Fits(1, 14592, 8, 48) && !Ub::Fits(1, 2048, 8, 0));
    EXPECT(Ub::Fits(28800, 2048, 46, 48) && !Ub::Fits(28800, 2048, 47, 48) && Ub::Fits(1, 7168, 6, 48));

    // registry: the operators register themselves under the reference's names
    auto& reg = OperatorRegistry::Instance();
    for (const char* name : {"MxQuantAllGather", "Ascend950MxFp8MatmulReduceScatter", "Ascend950DispatchFFNCombine",
                             "Ascend950Fp4MxAllToAllVGroupedMatmul", "DispatchGmmDequantSwiglu", "Ascend950Fp8MxAllGatherMatmul",
                             "Ascend950Fp4MxAllGatherMatmul", "Ascend950MxFp8MatmulAllToAll", "Ascend950Fp4MxMatmulReduceScatter",
                             "Ascend950Fp8MxAllToAllVGroupedMatmul", "Ascend950Fp8MxGroupedMatmulAllToAllV",
                             "Ascend950Fp4MxGroupedMatmulAllToAllV", "Ascend950MxFp8AllToAllMatmulSplitKUrma"}) {
        EXPECT(reg.CreateOperator(name) != nullptr);
    }
    EXPECT(reg.CreateOperator("NoSuchOperator") == nullptr);
    EXPECT(!reg.RegisterOperator("MxQuantAllGather", []() -> std::unique_ptr<CatccosOperator> { return nullptr; }));
    EXPECT(reg.CreateOperator("MxQuantAllGather") != nullptr);           // first registration kept

    // identifiers
    EXPECT(static_cast<int>(ASCEND950_DISPATCH_FFN_COMBINE) == 32 && static_cast<int>(MX_QUANT_ALLGATHER) == 24);
    EXPECT(static_cast<int>(TYPE_NUM) == 45);
    EXPECT(GetCommType("a5moe") == ASCEND950_DISPATCH_FFN_COMBINE && GetCommType("nope") == UNKNOWN);
    EXPECT(CommTypeOpNameMap.at(DISPATCH_GMM_DEQUANT_SWIGLU) == "DispatchGmmDequantSwiglu");
    EXPECT(CommTypeMap.size() == 41 && CommTypeOpNameMap.size() == 41);
    EXPECT(GetKernelFunc(ASCEND950_DISPATCH_FFN_COMBINE, BF16) != nullptr && GetKernelFunc(MATMUL_ALLREDUCE, FP16) == nullptr);

    // tiling validation of the FFN operator
    auto ffn = reg.CreateOperator("Ascend950DispatchFFNCombine");
    CocTilingParams t{};
    t.m = 512; t.k = 7168; t.n = 4096; t.m0 = 128; t.n0 = 256; t.k0 = 256; t.commInterval = 10;
    t.rankSize = 1; t.epSize = 1; t.expertNum = 16; t.topK = 6;
    EXPECT(ffn->ValidateCocTilingParams(1, t));
    EXPECT(!ffn->ValidateCocTilingParams(2, t));                          // rank mismatch
    CocTilingParams bad = t; bad.k = 7168 + 128;
    EXPECT(!ffn->ValidateCocTilingParams(1, bad));                        // K % 256
    bad = t; bad.n = 4096 + 256;
    EXPECT(!ffn->ValidateCocTilingParams(1, bad));                        // N % 512
    bad = t; bad.topK = 17;
    EXPECT(!ffn->ValidateCocTilingParams(1, bad));                        // topK > experts
    bad = t; bad.m0 = 0;
    EXPECT(!ffn->ValidateCocTilingParams(1, bad));                        // common check
    // the published workspace size equals the C ABI's (both restate the reference formula)
    EXPECT(ffn->GetWorkspaceSize(t) == catccos_ascend950_dispatch_ffn_combine_workspace_bytes(t.m, t.k, t.n, 16, 6, 1));
    t.m = 8192; t.expertNum = 256; t.topK = 8;
    EXPECT(ffn->GetWorkspaceSize(t) == catccos_ascend950_dispatch_ffn_combine_workspace_bytes(t.m, t.k, t.n, 256, 8, 1));
    EXPECT(ffn->GetSymmetricSize(t) == static_cast<size_t>(SHMEM_BUFF_BYTES) && catccos_ascend950_symmetric_bytes() == 1004ull * 1024 * 1024);

    // quantizer shape rule
    auto q = reg.CreateOperator("MxQuantAllGather");
    CocTilingParams qt{};
    qt.m = 4096; qt.n = 7168; qt.k = 1; qt.m0 = qt.n0 = qt.k0 = 1; qt.rankSize = 1;
    EXPECT(q->ValidateCocTilingParams(1, qt));
    qt.n = 7168 + 16;
    EXPECT(!q->ValidateCocTilingParams(1, qt));

    // KernelParams is move-only and owns its pointer array
    KernelParams p;
    uint8_t dummy[4];
    p.SetKernelParams(dummy, dummy + 1, dummy + 2, dummy + 3, dummy);
    EXPECT(p.customCount == 2 && p.customPtrs[0] == dummy + 3);
    KernelParams moved(std::move(p));
    EXPECT(moved.customCount == 2 && p.customPtrs == nullptr && p.ptrA == nullptr);

    // file helpers: offset writes, size-checked reads, overflow-checked sizes
    const std::string path = "/tmp/catccos_mx_host_test.bin";
    std::remove(path.c_str());
    std::vector<uint8_t> a(64, 7), b(64, 9), back(128);
    EXPECT(WriteFile(path, b.data(), 64, 64) && WriteFile(path, a.data(), 64, 0));
    EXPECT(ReadFile(path, back.data(), 128) && back[0] == 7 && back[64] == 9);
    EXPECT(!ReadFile(path, back.data(), 100));
    bool threw = false;
    try { ReadFileOrThrow("/tmp/definitely_missing_file.bin", back.data(), 1); } catch (const std::runtime_error&) { threw = true; }
    EXPECT(threw);
    threw = false;
    try { CheckedBufferSize({size_t{1} << 40, size_t{1} << 40}); } catch (const std::overflow_error&) { threw = true; }
    EXPECT(threw && CheckedBufferSize({3, 5, 7}) == 105);
    std::remove(path.c_str());
    EXPECT(Roundup<size_t>(513, 512) == 1024 && CeilDev(7168, 32) == 224 && IsNeedPadding(4, 100, 0, 32) && !IsNeedPadding(4, 128, 0, 32));

    std::cout << "host layer checks: PASS" << std::endl;
    return EXIT_SUCCESS;
}
