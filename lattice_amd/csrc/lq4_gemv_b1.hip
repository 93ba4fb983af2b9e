// Launchers of the batch-1 decode GEMV kernel (lq4_gemv_b1_kernel.hpp): plain, fused, LoRA factor inside the launch,
// and the lm_head pass with the top-k selection in the same launch.
#include "lq4_gemv_b1_kernel.hpp"

namespace lq4 {

namespace {

template <int RW, int SG>
void launch_cfg_topk(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, const TopkEpilogue& topk,
                     size_t lds, uint32_t waves, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, 64, kTopkMode, 4>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        attr_set = true;
    }
    hipLaunchKernelGGL((gemv_q4_b1<RW, SG, 64, kTopkMode, 4>), dim3((waves + 3) / 4), dim3(256), lds, stream, w, n, k, x,
                       y, LoraEpilogue{}, topk);
}

template <int RW, int SG, int SEG, int WAVES = kWaves>
void launch_cfg(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, const LoraEpilogue& lora,
                const GemvFusion* fusion, size_t lds, uint32_t waves, bool persistent, hipStream_t stream) {
    static bool attr_set[4] = {false, false, false, false};  // raise the dynamic-LDS cap once per instantiation
    const dim3 grid((waves + WAVES - 1) / WAVES), block(WAVES * 64);
    if constexpr (RW % 2 == 0 && SEG == 64) {
        if (fusion && fusion->epilogue == GemvFusion::kSiluMulPairs) {
            static bool attr_pairs = false;
            if (!attr_pairs) {
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kFusedPairsMode, WAVES>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 159 * 1024);
                attr_pairs = true;
            }
            hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kFusedPairsMode, WAVES>), grid, block, lds, stream, w, n, k, x, y,
                               lora, *fusion);
            return;
        }
    }
    if (fusion) {
        if (!attr_set[1]) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kFusedMode, WAVES>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 159 * 1024);
            attr_set[1] = true;
        }
        hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kFusedMode, WAVES>), grid, block, lds, stream, w, n, k, x, y, lora,
                           *fusion);
        return;
    }
    if (lora.rank && lora.a) {
        if (!attr_set[2]) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kLoraAMode, WAVES>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            attr_set[2] = true;
        }
        const dim3 grid_a(grid.x + lora.rank);  // the rank producer workgroups come first
        hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kLoraAMode, WAVES>), grid_a, block, lds, stream, w, n, k, x, y,
                           lora, NoFusion{});
        return;
    }
    if constexpr (RW > 1) {  // (one row per chunk: both row orders are the same)
        if (persistent) {
            if (!attr_set[3]) {
                (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kPlainAdjMode, WAVES>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                attr_set[3] = true;
            }
            hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, kPlainAdjMode, WAVES>), grid, block, lds, stream, w, n, k, x, y,
                               lora, NoFusion{});
            return;
        }
    }
    if (!attr_set[0]) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, kPlainMode, WAVES>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        attr_set[0] = true;
    }
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

// The lm_head pass that selects in its own launch serves four-wave workgroups over rows of one or
// more 64-block slabs (K of 2048 and up, not 512 or 1024), k up to 64, between k and 1024 workgroups.
bool plan_b1_topk(uint32_t n, uint32_t k, uint32_t topk, B1Plan* out, uint32_t* runs) {
    if (topk == 0 || topk > kSingleKernelMaxK || n == 0) return false;
    if (gemv_b1_lds_bytes(k) > 128 * 1024) return false;
    const B1Plan pl = plan_b1(n, k, 0, true, sizeof(TopkTailShared) + 64);
    if (pl.seg != 64) return false;
    const uint32_t grid = (pl.waves + 3) / 4;
    if (grid > 1024 || grid < topk) return false;
    *out = pl;
    *runs = (n + grid * 4 - 1) / (grid * 4);  // rows per wave; a workgroup's block is four times that
    return true;
}

}  // namespace

size_t gemv_b1_topk_scratch_bytes(uint32_t n, uint32_t k, uint32_t topk) {
    B1Plan pl;
    uint32_t runs;
    if (!plan_b1_topk(n, k, topk, &pl, &runs)) return 0;
    const size_t logits = (static_cast<size_t>(n) * sizeof(float) + 255) / 256 * 256;
    return logits + 1024 * sizeof(uint64_t) + static_cast<size_t>(topk_most_blocks(topk)) * runs * 4 * sizeof(Cand);
}

void launch_gemv_b1_topk(const uint8_t* w, uint32_t n, uint32_t k, const float* x, void* scratch, uint32_t* ticket,
                         uint32_t topk, float* out_logits, uint32_t* out_ids, hipStream_t stream) {
    B1Plan pl;
    uint32_t runs;
    if (!plan_b1_topk(n, k, topk, &pl, &runs)) return;  // the caller asked gemv_b1_topk_scratch_bytes first
    float* logits = static_cast<float*>(scratch);
    TopkEpilogue te;
    te.maxima = reinterpret_cast<uint64_t*>(static_cast<uint8_t*>(scratch) + (static_cast<size_t>(n) * sizeof(float) + 255) / 256 * 256);
    te.surv = reinterpret_cast<Cand*>(te.maxima + 1024);
    te.ticket = ticket;
    te.k = topk;
    te.out_logits = out_logits;
    te.out_ids = out_ids;
#define LQ4_B1T(RW_, SG_) launch_cfg_topk<RW_, SG_>(w, n, k, x, logits, te, pl.lds, pl.waves, stream)
    const uint32_t rw = pl.rw, sg = pl.sg;
    if (rw == 1) { if (sg == 1) LQ4_B1T(1, 1); else if (sg == 2) LQ4_B1T(1, 2); else LQ4_B1T(1, 3); }
    else if (rw == 2) { if (sg == 1) LQ4_B1T(2, 1); else if (sg == 2) LQ4_B1T(2, 2); else LQ4_B1T(2, 3); }
    else if (rw == 3) { if (sg == 1) LQ4_B1T(3, 1); else LQ4_B1T(3, 2); }
    else LQ4_B1T(4, 1);
#undef LQ4_B1T
}

}  // namespace lq4
