// "Ascend950DispatchFFNCombine" on one GPU: routing sort -> MX quantise + scatter -> GMM1 + SwiGLU +
// requant -> GMM2 -> weighted combine.  Host contract (buffer order, .bin names, workspace size,
// shape checks) follows examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_host.h:16-209.
#ifndef ASCEND950_DISPATCH_FFN_COMBINE_HOST_H
#define ASCEND950_DISPATCH_FFN_COMBINE_HOST_H

#include "catccos/detail/ascend950_moe_ready.hpp"
#include "op_common.h"

class Ascend950DispatchFFNCombineOperator : public CatccosOperator {
public:
    // AllocateDeviceSpace is where this operator loads its weights, so it is also where they are brought into the order
    // the fastest grouped kernels read (cmx_mx_pretile_weights, one pass): for the shapes that path covers, ptrB and the
    // W2 pointer then hold tiled weights and Launch calls the pre-tiled entry point, whose output has the same bits.
    static bool WeightsPretiled(const CocTilingParams& t) { return t.k % 512 == 0 && t.n % 1024 == 0; }

    static uint8_t* Pretile(uint8_t* w, uint32_t experts, uint32_t rows, uint32_t cols, int pairGateUp)
    {
        const size_t bytes = cmx_mx_pretiled_weight_bytes(experts, rows, cols, pairGateUp);
        uint8_t* tiled = mxrt::DeviceAlloc(bytes);
        MX_CHECK(cmx_mx_pretile_weights(w, tiled, experts, rows, cols, pairGateUp, nullptr));
        MX_CHECK(cmx_rt_stream_sync(nullptr));
        MX_CHECK(cmx_rt_free(w));
        return tiled;
    }

    // Buffer order after AllocateDeviceSpace:
    //   ptrA = x bf16 [m,k], ptrB = W1 [E,n,k], ptrC = out bf16 [m,k],
    //   custom = { W2 [E,k,n/2], expertIdx i32 [m,topK], probs f32 [m,topK], W1 scale [E,n,k/32], W2 scale [E,k,n/64] }
    void AllocateDeviceSpace(KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t experts = t.expertNum / t.epSize;
        const size_t k2 = t.n / 2, n2 = t.k;
        const size_t xBytes = static_cast<size_t>(t.m) * t.k * sizeof(uint16_t);
        const size_t w1Bytes = static_cast<size_t>(t.k) * t.n * experts;
        const size_t w2Bytes = k2 * n2 * experts;
        const size_t w1ScaleBytes = mxops::ScaleCols(t.k) * t.n * experts;
        const size_t w2ScaleBytes = mxops::ScaleCols(k2) * n2 * experts;
        const size_t routeBytes = static_cast<size_t>(t.m) * t.topK * sizeof(int32_t);
        auto file = [&](const char* stem) { return mxops::RankFile(dataFile, stem, rankId, false); };
        const bool fromFiles = !dataFile.empty();
        uint8_t* x = nullptr;
        if (fromFiles) {
            x = mxops::DeviceBufferFromFile(xBytes, file("in_routing_matrix_a"));
        } else {
            std::vector<uint16_t> ones(static_cast<size_t>(t.m) * t.k, 0x3F80);     // bf16 1.0
            x = mxops::DeviceBufferFromValues(ones.data(), xBytes);
        }
        uint8_t* w1 = mxops::DeviceBufferFromFile(w1Bytes, fromFiles ? file("in_gmm_matrix_b") : "", 1);
        uint8_t* w2 = mxops::DeviceBufferFromFile(w2Bytes, fromFiles ? file("in_gmm_matrix_b2") : "", 1);
        // scales, routing and gate weights have no defaults: they are always read
        uint8_t* w1Scale = mxops::DeviceBufferFromFile(w1ScaleBytes, file("in_gmm_matrix_b_scale"));
        uint8_t* w2Scale = mxops::DeviceBufferFromFile(w2ScaleBytes, file("in_gmm_matrix_b2_scale"));
        uint8_t* expertIdx = mxops::DeviceBufferFromFile(routeBytes, file("in_routing_expert_idx"));
        uint8_t* probs = mxops::DeviceBufferFromFile(routeBytes, file("in_gather_gate_weight"));
        uint8_t* out = mxrt::DeviceAlloc(xBytes);
        MX_CHECK(cmx_rt_memset(out, 0, xBytes));
        if (WeightsPretiled(t)) {
            w1 = Pretile(w1, static_cast<uint32_t>(experts), t.n, t.k, 1);
            w2 = Pretile(w2, static_cast<uint32_t>(experts), static_cast<uint32_t>(n2), static_cast<uint32_t>(k2), 0);
        }
        params.SetKernelParams(x, w1, out, w2, expertIdx, probs, w1Scale, w2Scale);
    }

    void WriteResultFile(const KernelParams& params, const CocTilingParams& t, uint32_t rankId, std::string dataFile) override
    {
        const size_t outBytes = static_cast<size_t>(t.m) * t.k * sizeof(uint16_t);
        mxops::DeviceBufferToFile(params.ptrC, outBytes, mxops::RankFile(dataFile, "output", rankId, false));
    }

    // Ten 512-byte-aligned regions; equals the reference operator's figure for the same arguments.
    size_t GetWorkspaceSize(const CocTilingParams& t) override
    {
        using Ready = Catccos::Detail::Ascend950MoeReady;
        const size_t experts = t.expertNum / t.epSize;
        const size_t ep = t.rankSize;
        const size_t rows = static_cast<size_t>(t.m) * t.rankSize * t.topK;
        const size_t meta = ep * ep * experts * sizeof(int32_t);
        const size_t half = t.n / 2;
        auto al = [](size_t b) { return RoundUp<size_t>(b, 512); };
        return al(RoundUp<size_t>(t.m, 256) * t.topK * sizeof(int32_t)) + al(rows * t.k * sizeof(uint16_t)) + al(meta) +
               al(rows * t.k) + al(rows * mxops::ScaleCols(t.k)) +
               Ready::SwigluRegionBytes(rows * half * sizeof(uint16_t), static_cast<uint32_t>(experts)) + al(rows * half) +
               al(rows * mxops::ScaleCols(half)) +
               Ready::DispatchRegionBytes(rows * t.k * sizeof(uint16_t), static_cast<uint32_t>(ep), static_cast<uint32_t>(experts)) +
               al(meta);
    }

    CocCommType GetActualKernelType(const CocTilingParams&) override { return CocCommType::ASCEND950_DISPATCH_FFN_COMBINE; }

    bool CheckCocTilingParams(uint32_t rankSize, const CocTilingParams& t) override
    {
        if (!CheckMoeCocTilingParams(t)) {
            return false;
        }
        if (t.topK > t.expertNum) {
            std::cerr << "TopK must not exceed the global expert count" << std::endl;
            return false;
        }
        if (rankSize != t.epSize) {
            std::cerr << "Ascend950DispatchFFNCombine requires rankSize == epSize" << std::endl;
            return false;
        }
        if (rankSize != 1) {
            std::cerr << "Ascend950DispatchFFNCombine: this build runs one device's share (rankSize 1)" << std::endl;
            return false;
        }
        // per-rank peer staging bound of the reference (kept so the same shapes are accepted and rejected)
        const uint32_t kLoop = CeilDev(t.k, t.k0);
        const int32_t maxPeerMemPerRank = IPC_BUFF_MAX_SIZE / INPUT_DTYPE / rankSize / MAX_BLOCK_COUNT;
        if (static_cast<uint64_t>(t.commInterval) * t.m0 * t.k0 * kLoop >= static_cast<uint64_t>(maxPeerMemPerRank)) {
            return false;
        }
        if (t.k % 256 != 0 || t.n % 512 != 0) {
            std::cerr << "MXFP8 FFN requires K % 256 == 0 and N % 512 == 0" << std::endl;
            return false;
        }
        const size_t expandedM = static_cast<size_t>(t.m) * t.topK;
        const size_t symmetricBytes = RoundUp<size_t>(expandedM * t.k * sizeof(uint16_t), 512) +
                                      RoundUp<size_t>(expandedM * RoundUp<size_t>(t.k + mxops::ScaleCols(t.k), 32), 512) +
                                      RoundUp<size_t>(static_cast<size_t>(rankSize) * rankSize * (t.expertNum / rankSize) * sizeof(int32_t), 512);
        if (symmetricBytes > static_cast<size_t>(SHMEM_BUFF_BYTES)) {
            std::cerr << "Packed input and BF16 return regions exceed symmetric buffer capacity" << std::endl;
            return false;
        }
        return true;
    }

    // launch order of the reference main: (A, W1, W1 scale, W2, W2 scale, out, expertIdx, probs, workspace, symmetric)
    static int Launch(void* stream, const KernelParams& p, uint8_t* out, uint8_t* workspace, uint8_t* symmetric,
                      const CocTilingParams& t)
    {
        if (WeightsPretiled(t)) {
            if (t.rankSize != 1) {
                return CMX_EINVAL;
            }
            return cmx_dispatch_ffn_combine_pretiled(stream, p.ptrA, p.customPtrs[1], p.customPtrs[2], p.ptrB, p.customPtrs[3],
                                                     p.customPtrs[0], p.customPtrs[4], out, workspace, t.m, t.k, t.n,
                                                     t.expertNum / t.epSize, t.topK);
        }
        return catccos_ascend950_dispatch_ffn_combine(0, stream, 0, p.ptrA, p.customPtrs[1], p.customPtrs[2], p.ptrB,
                                                      p.customPtrs[3], p.customPtrs[0], p.customPtrs[4], out, workspace, symmetric,
                                                      t.m, t.k, t.n, t.expertNum / t.epSize, t.topK, static_cast<int>(t.rankSize));
    }
};

REGISTER_OPERATOR("Ascend950DispatchFFNCombine", Ascend950DispatchFFNCombineOperator);

#endif  // ASCEND950_DISPATCH_FFN_COMBINE_HOST_H
