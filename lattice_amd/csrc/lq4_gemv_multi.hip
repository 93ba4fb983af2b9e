// Several projections of one activation vector in one launch (q, k and v of an attention layer; the q and v of a
// LoRA adapter): the batch-1 GEMV kernel walks the rows of the matrices stacked one under the other, so the launch,
// the staging of x and the start of the stream are paid once.  The LoRA factors t_v = A_v . x of every view that has
// an adapter come from one launch as well.
#include "lq4_gemv_b1_kernel.hpp"

namespace lq4 {

namespace {

// t_v[row, j] = A_v[j, :] . x[row, :] for every view v with an adapter: one workgroup per (j, v, row), the summation
// of lora_a_kernel (256 threads, eight elements a step, wave sums, then the four waves' sums pairwise).
__global__ __launch_bounds__(256) void lora_a_views_kernel(LoraAViews av, uint32_t d_in, const float* __restrict__ x,
                                                           uint32_t x_stride) {
    const uint32_t j = blockIdx.x, v = blockIdx.y, row = blockIdx.z;
    const uint32_t rank = av.rank[v];
    if (j >= rank) return;  // uniform across the workgroup
    const float* xr = x + static_cast<size_t>(row) * x_stride;
    float p = 0.0f;
    if (av.a_is_f16[v]) {
        const _Float16* ar = static_cast<const _Float16*>(av.a[v]) + static_cast<size_t>(j) * d_in;
        struct alignas(16) H8 { _Float16 v[8]; };
        for (uint32_t kk = threadIdx.x * 8; kk < d_in; kk += 256 * 8) {
            const H8 h = *reinterpret_cast<const H8*>(ar + kk);
            const float4 x0 = *reinterpret_cast<const float4*>(xr + kk), x1 = *reinterpret_cast<const float4*>(xr + kk + 4);
            p = fmaf(static_cast<float>(h.v[0]), x0.x, p); p = fmaf(static_cast<float>(h.v[1]), x0.y, p);
            p = fmaf(static_cast<float>(h.v[2]), x0.z, p); p = fmaf(static_cast<float>(h.v[3]), x0.w, p);
            p = fmaf(static_cast<float>(h.v[4]), x1.x, p); p = fmaf(static_cast<float>(h.v[5]), x1.y, p);
            p = fmaf(static_cast<float>(h.v[6]), x1.z, p); p = fmaf(static_cast<float>(h.v[7]), x1.w, p);
        }
    } else {
        const float* ar = static_cast<const float*>(av.a[v]) + static_cast<size_t>(j) * d_in;
        for (uint32_t kk = threadIdx.x * 8; kk < d_in; kk += 256 * 8) {
            const float4 a0 = *reinterpret_cast<const float4*>(ar + kk), a1 = *reinterpret_cast<const float4*>(ar + kk + 4);
            const float4 x0 = *reinterpret_cast<const float4*>(xr + kk), x1 = *reinterpret_cast<const float4*>(xr + kk + 4);
            p = fmaf(a0.x, x0.x, p); p = fmaf(a0.y, x0.y, p); p = fmaf(a0.z, x0.z, p); p = fmaf(a0.w, x0.w, p);
            p = fmaf(a1.x, x1.x, p); p = fmaf(a1.y, x1.y, p); p = fmaf(a1.z, x1.z, p); p = fmaf(a1.w, x1.w, p);
        }
    }
    p = wave_sum(p);
    __shared__ float part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = p;
    __syncthreads();
    if (threadIdx.x == 0) av.t[v][static_cast<size_t>(row) * rank + j] = (part[0] + part[1]) + (part[2] + part[3]);
}

template <int RW, int SG, int SEG, int MODE>
void launch_multi_cfg(const MultiViews& mv, uint32_t n, uint32_t k, const float* x, const LoraEpilogue& lora, size_t lds,
                      uint32_t waves, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q4_b1<RW, SG, SEG, MODE, 4>), 160 * 1024);
    // (producer workgroups, if any, come first)
    hipLaunchKernelGGL((gemv_q4_b1<RW, SG, SEG, MODE, 4>), dim3((waves + 3) / 4 + lora.rank), dim3(256), lds, stream,
                       static_cast<const uint8_t*>(nullptr), n, k, x, static_cast<float*>(nullptr), lora, mv);
}

}  // namespace

// One launch serves the views when the activations fit the kernel's LDS staging and, for rows shorter than a slab
// (two or four rows side by side in a wave), no group of side-by-side rows straddles two views.
bool gemv_multi_serves(const MultiViews& mv, uint32_t k) {
    if (k == 0 || k % kBlockWeights || gemv_b1_lds_bytes(k) > 128 * 1024) return false;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t side = nb == 32 ? 2 : nb == 16 ? 4 : 1;
    for (uint32_t v = 0; v < mv.count; ++v)
        if ((mv.begin[v + 1] - mv.begin[v]) % side) return false;
    return mv.count >= 1 && mv.count <= static_cast<uint32_t>(kMaxViews) && mv.begin[mv.count] != 0;
}

void launch_gemv_multi(const MultiViews& mv, uint32_t k, const float* x, const LoraEpilogue* in_launch, hipStream_t stream) {
    const uint32_t n = mv.begin[mv.count];
    const LoraEpilogue lora = in_launch ? *in_launch : LoraEpilogue{};
    const B1Plan pl = plan_b1(n, k, lora.rank, true, 0);
    const uint32_t seg = pl.seg, rw = pl.rw, sg = pl.sg;
#define LQ4_MULTI(RW_, SG_, SEG_)                                                                              \
    do {                                                                                                       \
        if (in_launch) launch_multi_cfg<RW_, SG_, SEG_, kMultiLoraAMode>(mv, n, k, x, lora, pl.lds, pl.waves, stream); \
        else launch_multi_cfg<RW_, SG_, SEG_, kMultiMode>(mv, n, k, x, lora, pl.lds, pl.waves, stream);        \
    } while (0)
    if (seg == 32) {
        if (rw == 1) LQ4_MULTI(1, 1, 32); else if (rw == 2) LQ4_MULTI(2, 1, 32); else if (rw == 3) LQ4_MULTI(3, 1, 32); else LQ4_MULTI(4, 1, 32);
    } else if (seg == 16) {
        if (rw == 1) LQ4_MULTI(1, 1, 16); else if (rw == 2) LQ4_MULTI(2, 1, 16); else if (rw == 3) LQ4_MULTI(3, 1, 16); else LQ4_MULTI(4, 1, 16);
    } else if (rw == 1) {
        if (sg == 1) LQ4_MULTI(1, 1, 64); else if (sg == 2) LQ4_MULTI(1, 2, 64); else LQ4_MULTI(1, 3, 64);
    } else if (rw == 2) {
        if (sg == 1) LQ4_MULTI(2, 1, 64); else if (sg == 2) LQ4_MULTI(2, 2, 64); else LQ4_MULTI(2, 3, 64);
    } else if (rw == 3) {
        if (sg == 1) LQ4_MULTI(3, 1, 64); else LQ4_MULTI(3, 2, 64);
    } else {
        LQ4_MULTI(4, 1, 64);
    }
#undef LQ4_MULTI
}

void launch_lora_a_views(const LoraAViews& av, uint32_t d_in, const float* x, uint32_t x_stride, uint32_t rows,
                         hipStream_t stream) {
    uint32_t most = 0;
    for (uint32_t v = 0; v < av.count; ++v) most = av.rank[v] > most ? av.rank[v] : most;
    if (!most) return;
    hipLaunchKernelGGL(lora_a_views_kernel, dim3(most, av.count, rows), dim3(256), 0, stream, av, d_in, x, x_stride);
}

}  // namespace lq4
