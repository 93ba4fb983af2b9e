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

// The same for rows that are whole, 16-byte aligned float4s: 16-byte accesses, the first kKeep float4s
// of a thread (rows up to 4096 wide have no more) stay in registers between the two passes, and their
// gamma is requested before the reduction, so a row costs one memory round trip instead of three.
__global__ __launch_bounds__(256) void residual_add_norm_vec_kernel(const float4* __restrict__ base,
                                                                    const float4* __restrict__ delta,
                                                                    const float4* __restrict__ gamma,
                                                                    uint32_t hidden4, float hidden_f, float eps,
                                                                    float4* residual_out,
                                                                    float4* __restrict__ normed_out) {
    constexpr int kKeep = 4;
    __shared__ float red[4];
    const size_t off = static_cast<size_t>(blockIdx.x) * hidden4;
    auto load_v = [&](uint32_t i) {
        float4 v = base[off + i];
        if (delta) {
            const float4 d = delta[off + i];
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        return v;
    };
    auto sq = [](const float4 v, float acc) { return fmaf(v.w, v.w, fmaf(v.z, v.z, fmaf(v.y, v.y, fmaf(v.x, v.x, acc)))); };
    auto emit = [&](uint32_t i, const float4 v, const float4 g, float inv_rms) {
        if (residual_out) residual_out[off + i] = v;
        float4 o;
        o.x = v.x * inv_rms * (1.0f + g.x); o.y = v.y * inv_rms * (1.0f + g.y);
        o.z = v.z * inv_rms * (1.0f + g.z); o.w = v.w * inv_rms * (1.0f + g.w);
        normed_out[off + i] = o;
    };
    float4 v[kKeep], g[kKeep];
#pragma unroll
    for (int c = 0; c < kKeep; ++c) {
        const uint32_t i = threadIdx.x + 256 * c;
        const uint32_t ic = i < hidden4 ? i : 0;  // clamped: no branch between these loads and their use
        v[c] = load_v(ic);
        g[c] = gamma[ic];
    }
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < kKeep; ++c)
        if (threadIdx.x + 256 * c < hidden4) ss = sq(v[c], ss);
    for (uint32_t i = threadIdx.x + 256 * kKeep; i < hidden4; i += 256) ss = sq(load_v(i), ss);
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv_rms = 1.0f / sqrtf(total / hidden_f + eps);
#pragma unroll
    for (int c = 0; c < kKeep; ++c) {
        const uint32_t i = threadIdx.x + 256 * c;
        if (i < hidden4) emit(i, v[c], g[c], inv_rms);
    }
    for (uint32_t i = threadIdx.x + 256 * kKeep; i < hidden4; i += 256) emit(i, load_v(i), gamma[i], inv_rms);
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

// The shared expert's sigmoid gate and its add onto the routed experts' sum (apply_shared_expert,
// crates/inference/src/model/qwen35/moe.rs:201-207 and 242-244; moe_shared_gate_add,
// shaders/qwen35.metal:2379-2392): one workgroup per token computes g = sigmoid(x . gate) and then
// y = fma(g, shared_out, y) over the token's row.
__global__ __launch_bounds__(256) void moe_shared_gate_add_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ gate,
                                                                  const float* __restrict__ shared_out,
                                                                  uint32_t hidden, float* y) {
    __shared__ float red[4];
    const size_t off = static_cast<size_t>(blockIdx.x) * hidden;
    float dot = 0.0f;
    for (uint32_t i = threadIdx.x; i < hidden; i += 256) dot = fmaf(x[off + i], gate[i], dot);
    dot = wave_sum(dot);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = dot;
    __syncthreads();
    const float logit = (red[0] + red[1]) + (red[2] + red[3]);
    const float g = 1.0f / (1.0f + expf(-logit));
    for (uint32_t i = threadIdx.x; i < hidden; i += 256) y[off + i] = fmaf(g, shared_out[off + i], y[off + i]);
}

}  // namespace

void launch_moe_shared_gate_add(const float* x, const float* gate, const float* shared_out, uint32_t hidden,
                                uint32_t tokens, float* y, hipStream_t stream) {
    hipLaunchKernelGGL(moe_shared_gate_add_kernel, dim3(tokens), dim3(256), 0, stream, x, gate, shared_out, hidden, y);
}

void launch_residual_add_norm(const float* base, const float* delta, const float* gamma, uint32_t hidden,
                              uint32_t rows, float eps, float* residual_out, float* normed_out, hipStream_t stream) {
    const auto aligned = [](const void* p) { return p == nullptr || reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (hidden % 4 == 0 && aligned(base) && aligned(delta) && aligned(gamma) && aligned(residual_out) &&
        aligned(normed_out)) {
        hipLaunchKernelGGL(residual_add_norm_vec_kernel, dim3(rows), dim3(256), 0, stream,
                           reinterpret_cast<const float4*>(base), reinterpret_cast<const float4*>(delta),
                           reinterpret_cast<const float4*>(gamma), hidden / 4, static_cast<float>(hidden), eps,
                           reinterpret_cast<float4*>(residual_out), reinterpret_cast<float4*>(normed_out));
        return;
    }
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
