// Launchers of the batch-1 decode GEMV kernel (lq4_gemv_b1_kernel.hpp): plain, fused, LoRA factor inside the launch.
#include "lq4_gemv_b1_kernel.hpp"

namespace lq4 {

namespace {

template <int RW, int SG, int SEG, int WAVES = kWaves>
void launch_cfg(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, const LoraEpilogue& lora,
                const GemvFusion* fusion, size_t lds, uint32_t waves, bool persistent, hipStream_t stream) {
    static LdsCapOnce cap[4];  // one per kernel mode of this instantiation
    const dim3 grid((waves + WAVES - 1) / WAVES), block(WAVES * 64);
    if constexpr (RW % 2 == 0 && SEG == 64) {
        if (fusion && fusion->epilogue == GemvFusion::kSiluMulPairs) {
            static LdsCapOnce cap_pairs;
            cap_pairs.raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kFusedPairsMode, WAVES>), 159 * 1024);
            hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kFusedPairsMode, WAVES>), grid, block, lds, stream, w, n, k, x, y,
                               lora, *fusion);
            return;
        }
    }
    if (fusion) {
        cap[1].raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kFusedMode, WAVES>), 159 * 1024);
        hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kFusedMode, WAVES>), grid, block, lds, stream, w, n, k, x, y, lora,
                           *fusion);
        return;
    }
    if (lora.rank && lora.a) {
        cap[2].raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kLoraAMode, WAVES>), 160 * 1024);
        const dim3 grid_a(grid.x + lora.rank);  // the rank producer workgroups come first
        hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kLoraAMode, WAVES>), grid_a, block, lds, stream, w, n, k, x, y,
                           lora, NoFusion{});
        return;
    }
    if constexpr (RW > 1) {  // (one row per chunk: both row orders are the same)
        if (persistent) {
            cap[3].raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kPlainAdjMode, WAVES>), 160 * 1024);
            hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kPlainAdjMode, WAVES>), grid, block, lds, stream, w, n, k, x, y,
                               lora, NoFusion{});
            return;
        }
    }
    cap[0].raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kPlainMode, WAVES>), 160 * 1024);
    hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kPlainMode, WAVES>), grid, block, lds, stream, w, n, k, x, y, lora,
                       NoFusion{});
}

void launch_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, const LoraEpilogue& lora,
               const GemvFusion* fusion, hipStream_t stream);

}  // namespace

size_t gemv_b1_lds_bytes(uint32_t k) { return static_cast<size_t>(k / kBlockWeights) * kXPitch * 4; }

// The kSiluMulPairs epilogue needs rows of 64 lanes (any block count but 16 and 32, which put rows side by side).
bool gemv_b1_pairs_served(uint32_t n, uint32_t k) {
    const uint32_t nb = k / kBlockWeights;
    return n >= 2 && n % 2 == 0 && nb != 16 && nb != 32;
}

void launch_gemv_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y,
                    const LoraEpilogue& lora, hipStream_t stream) {
    launch_b1(w, n, k, x, y, lora, nullptr, stream);
}

void launch_gemv_b1_fused(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y,
                          const LoraEpilogue& lora, const GemvFusion& fusion, hipStream_t stream) {
    launch_b1(w, n, k, x, y, lora, &fusion, stream);
}

namespace {

void launch_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, const LoraEpilogue& lora,
               const GemvFusion* fusion, hipStream_t stream) {
    const bool pairs = fusion && fusion->epilogue == GemvFusion::kSiluMulPairs;
    const B1Plan pl = plan_b1(n, k, (lora.rank && lora.a && !fusion) ? lora.rank : 0, false, 0, pairs);
    const size_t lds = pl.lds;
    const uint32_t seg = pl.seg, wg_waves = pl.wg_waves, waves = pl.waves, rw = pl.rw, sg = pl.sg;

#define LQ4_B1(RW_, SG_, SEG_) launch_cfg<RW_, SG_, SEG_>(w, n, k, x, y, lora, fusion, lds, waves, pl.persistent, stream)
#define LQ4_B1W(RW_, SG_) launch_cfg<RW_, SG_, 64, 8>(w, n, k, x, y, lora, fusion, lds, waves, pl.persistent, stream)
    if (seg == 32) {
        if (rw == 1) LQ4_B1(1, 1, 32); else if (rw == 2) LQ4_B1(2, 1, 32); else if (rw == 3) LQ4_B1(3, 1, 32); else LQ4_B1(4, 1, 32);
    } else if (seg == 16) {
        if (rw == 1) LQ4_B1(1, 1, 16); else if (rw == 2) LQ4_B1(2, 1, 16); else if (rw == 3) LQ4_B1(3, 1, 16); else LQ4_B1(4, 1, 16);
    } else if (wg_waves == 8) {  // K 4096..8192: two to four slabs
        if (rw == 1) { if (sg == 2) LQ4_B1W(1, 2); else LQ4_B1W(1, 3); }
        else if (rw == 2) { if (sg == 2) LQ4_B1W(2, 2); else LQ4_B1W(2, 3); }
        else if (rw == 3) LQ4_B1W(3, 2);
        else LQ4_B1W(4, 1);
    } else if (rw == 1) {
        if (sg == 1) LQ4_B1(1, 1, 64); else if (sg == 2) LQ4_B1(1, 2, 64); else LQ4_B1(1, 3, 64);
    } else if (rw == 2) {
        if (sg == 1) LQ4_B1(2, 1, 64); else if (sg == 2) LQ4_B1(2, 2, 64); else LQ4_B1(2, 3, 64);
    } else if (rw == 3) {
        if (sg == 1) LQ4_B1(3, 1, 64); else LQ4_B1(3, 2, 64);
    } else {
        LQ4_B1(4, 1, 64);
    }
#undef LQ4_B1W
#undef LQ4_B1
}

}  // namespace

}  // namespace lq4
