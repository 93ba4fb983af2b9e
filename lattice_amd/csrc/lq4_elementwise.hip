// Stand-alone forms of the elementwise steps either side of the decode GEMVs, for any number
// of rows: residual add + shifted RMSNorm (shaders/qwen35.metal:739-767, 2219-2249; CPU form
// model/qwen35/norm.rs:6-23), silu(gate) * up (shaders/qwen35.metal:712-722) and the
// add-into-residual-and-copy that ends a layer (shaders/qwen35.metal:2255-2266).  At batch 1 the
// same steps run inside the GEMV kernel instead (gemv_q4_b1<.., FUSED>); these kernels serve
// prefill rows and shapes the fused kernel does not take.
#include "lq4_internal.hpp"

namespace lq4 {

namespace {

// One workgroup per row.  v = base + delta is recomputed in the second pass rather than kept:
// it is bit-identical and the row is L2-resident.
__global__ __launch_bounds__(256) void residual_add_norm_kernel(const float* __restrict__ base,
                                                                const float* __restrict__ delta,
                                                                const float* __restrict__ gamma, uint32_t hidden,
                                                                float eps, float* residual_out,
                                                                float* __restrict__ normed_out) {
    __shared__ float red[4];
    const size_t off = static_cast<size_t>(blockIdx.x) * hidden;
    float ss = 0.0f;
    for (uint32_t i = threadIdx.x; i < hidden; i += 256) {
        const float v = delta ? base[off + i] + delta[off + i] : base[off + i];
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv_rms = 1.0f / sqrtf(total / static_cast<float>(hidden) + eps);
    for (uint32_t i = threadIdx.x; i < hidden; i += 256) {
        const float v = delta ? base[off + i] + delta[off + i] : base[off + i];
        if (residual_out) residual_out[off + i] = v;
        normed_out[off + i] = v * inv_rms * (1.0f + gamma[i]);
    }
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float* gate_up, uint32_t count, float* out,
                                                       uint32_t out_stride) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    const size_t in = static_cast<size_t>(blockIdx.y) * 2 * count;
    const float gate = gate_up[in + i], up = gate_up[in + count + i];
    out[static_cast<size_t>(blockIdx.y) * out_stride + i] = gate / (1.0f + expf(-gate)) * up;
}

__global__ __launch_bounds__(256) void add_and_copy_kernel(const float* __restrict__ src, float* residual, float* dst,
                                                           size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= count) return;
    const float r = residual[i] + src[i];
    residual[i] = r;
    if (dst) dst[i] = r;
}

}  // namespace

void launch_residual_add_norm(const float* base, const float* delta, const float* gamma, uint32_t hidden,
                              uint32_t rows, float eps, float* residual_out, float* normed_out, hipStream_t stream) {
    hipLaunchKernelGGL(residual_add_norm_kernel, dim3(rows), dim3(256), 0, stream, base, delta, gamma, hidden, eps,
                       residual_out, normed_out);
}

void launch_silu_mul(const float* gate_up, uint32_t count, uint32_t rows, float* out, uint32_t out_stride,
                     hipStream_t stream) {
    hipLaunchKernelGGL(silu_mul_kernel, dim3((count + 255) / 256, rows), dim3(256), 0, stream, gate_up, count, out,
                       out_stride);
}

void launch_add_and_copy(const float* src, float* residual, float* dst, size_t count, hipStream_t stream) {
    hipLaunchKernelGGL(add_and_copy_kernel, dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, stream, src,
                       residual, dst, count);
}

}  // namespace lq4
