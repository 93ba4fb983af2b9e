// MoE routing and grouped expert GEMV over native Q4 expert tensors.
//
// Routing restates compute_router_probs / select_top_k / renormalize_selected
// (crates/inference/src/model/qwen35/moe.rs:39-125).  The expert pass groups the
// (token, slot) pairs by expert so each routed expert's blocks stream from HBM once
// for all of its tokens, then combines per token in slot order, the order
// accumulate_routed_experts uses (moe.rs:127-190).
#include "lq4_internal.hpp"
#include "lq4_moe_route_dev.hpp"

namespace lq4 {

namespace {

constexpr int kMaxExperts = 1024;

// Router of one token per wave: see route_one_token.  The routing table has `out_stride` slots per token.
// With a shared expert (`shared_gate` not null) the wave also fills slot `top_k`: expert id `num_experts` (the
// grouped kernels read that expert from the shared expert's own tensors) with weight sigmoid(x . shared_gate).
template <int kPerLane>
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ logits, uint32_t tokens,
                                                       uint32_t num_experts, uint32_t top_k,
                                                       int32_t* __restrict__ ids, float* __restrict__ weights,
                                                       uint32_t out_stride, const float* __restrict__ x,
                                                       const float* __restrict__ shared_gate, uint32_t hidden) {
    __shared__ float s_ev[64 * kPerLane];
    const uint32_t t = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    float dot = 0.0f;
    if (shared_gate != nullptr) {
        const float* xr = x + static_cast<size_t>(t) * hidden;
        if (hidden % 4 == 0 && reinterpret_cast<uintptr_t>(xr) % 16 == 0 && reinterpret_cast<uintptr_t>(shared_gate) % 16 == 0) {
            // 16-byte loads, four rounds in flight together (a dependent chain of single loads made this the
            // longest launch of the layer)
            const float4* x4 = reinterpret_cast<const float4*>(xr);
            const float4* g4 = reinterpret_cast<const float4*>(shared_gate);
            const uint32_t n4 = hidden / 4;
            float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint32_t i0 = lane; i0 < n4; i0 += 4 * 64) {
                float4 xv[4], gv[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t i = i0 + r * 64 < n4 ? i0 + r * 64 : lane;
                    xv[r] = x4[i];
                    gv[r] = g4[i];
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (i0 + r * 64 >= n4) continue;
                    part[r] = fmaf(xv[r].x, gv[r].x, part[r]);
                    part[r] = fmaf(xv[r].y, gv[r].y, part[r]);
                    part[r] = fmaf(xv[r].z, gv[r].z, part[r]);
                    part[r] = fmaf(xv[r].w, gv[r].w, part[r]);
                }
            }
            dot = (part[0] + part[1]) + (part[2] + part[3]);
        } else {
            for (uint32_t i = lane; i < hidden; i += 64) dot = fmaf(xr[i], shared_gate[i], dot);
        }
    }
    int32_t id;
    float w;
    route_one_token<kPerLane>(logits + static_cast<size_t>(t) * num_experts, num_experts, top_k, lane, s_ev, id, w);
    if (lane < top_k) {
        ids[t * out_stride + lane] = id;
        weights[t * out_stride + lane] = w;
    }
    if (shared_gate != nullptr) {
        dot = wave_sum(dot);
        if (lane == 0) {
            ids[t * out_stride + top_k] = static_cast<int32_t>(num_experts);
            weights[t * out_stride + top_k] = 1.0f / (1.0f + expf(-dot));
        }
    }
}

// Stable grouping of the (token, slot) pairs by expert: counts, offsets (exclusive prefix) and `order`, in which the
// pairs of one expert stay in ascending pair index.  One workgroup of sixteen waves:
//   1. a histogram of the experts (LDS integer atomics: the totals do not depend on the order of arrival) and its
//      exclusive scan, which also becomes every expert's cursor;
//   2. rounds of 1024 pairs, a wave per 64 of them: the lanes of a wave that share an expert rank themselves with
//      ballots (registers only, one turn per distinct expert of the wave) and the first of them notes how many they
//      are in a [wave][expert] table; a thread per expert turns its column into an exclusive prefix over the waves and
//      moves the expert's cursor on; every pair then knows its place: cursor + pairs of its expert in the waves
//      before it + its rank in its wave.
// (An earlier form of four waves that walked their segments with a cursor in LDS per ballot turn needed 34 us for 576
// pairs and 54 us for 1152; this one about 5.)
constexpr int kGroupThreads = 1024, kGroupWaves = kGroupThreads / 64;

__global__ __launch_bounds__(kGroupThreads) void moe_group_kernel(const int32_t* __restrict__ ids, uint32_t pairs,
                                                                  uint32_t num_experts, int32_t* __restrict__ counts,
                                                                  int32_t* __restrict__ offsets,
                                                                  int32_t* __restrict__ order) {
    __shared__ int32_t s_cur[kMaxExperts + 2];   // counts, then the cursor of every expert
    __shared__ int32_t s_base[kMaxExperts + 2];  // the cursor at the start of the round
    __shared__ int32_t s_wsum[kGroupWaves];
    __shared__ uint16_t s_tbl[kGroupWaves][kMaxExperts + 2];  // pairs of an expert in a wave, then in the waves before it
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    auto valid_id = [&](int32_t e) { return e >= 0 && e < static_cast<int32_t>(num_experts); };
    for (uint32_t e = tid; e < num_experts; e += kGroupThreads) s_cur[e] = 0;
    __syncthreads();
    for (uint32_t p = tid; p < pairs; p += kGroupThreads) {
        const int32_t e = ids[p];
        if (valid_id(e)) atomicAdd(&s_cur[e], 1);
    }
    __syncthreads();
    int32_t carry = 0;
    for (uint32_t base = 0; base < num_experts; base += kGroupThreads) {  // (uniform)
        const uint32_t e = base + tid;
        const int32_t c = e < num_experts ? s_cur[e] : 0;
        int32_t incl = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int32_t up = __shfl_up(incl, d, 64);
            if (static_cast<int>(lane) >= d) incl += up;
        }
        if (lane == 63) s_wsum[wave] = incl;
        __syncthreads();
        int32_t before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kGroupWaves; ++w) {
            before += static_cast<uint32_t>(w) < wave ? s_wsum[w] : 0;
            total += s_wsum[w];
        }
        __syncthreads();  // (s_wsum is written again in the next turn)
        if (e < num_experts) {
            const int32_t excl = carry + before + incl - c;
            counts[e] = c;
            offsets[e] = excl;
            s_cur[e] = excl;
        }
        carry += total;
    }
    if (tid == 0) offsets[num_experts] = carry;
    for (uint32_t p0 = 0; p0 < pairs; p0 += kGroupThreads) {  // (uniform)
        for (int w = 0; w < kGroupWaves; ++w)
            for (uint32_t e = tid; e < num_experts; e += kGroupThreads) s_tbl[w][e] = 0;
        __syncthreads();  // (also: the cursors are in place)
        const uint32_t p = p0 + tid;
        const int32_t e = p < pairs ? ids[p] : -1;
        const bool valid = valid_id(e);
        int32_t rank = 0;
        unsigned long long active = __ballot(valid);
        while (active) {  // (uniform in the wave)
            const int leader = __ffsll(static_cast<long long>(active)) - 1;
            const int32_t le = __shfl(e, leader, 64);
            const bool mine = valid && e == le;
            const unsigned long long m = __ballot(mine);
            if (mine) rank = __popcll(m & ((1ull << lane) - 1ull));
            if (static_cast<int>(lane) == leader) s_tbl[wave][le] = static_cast<uint16_t>(__popcll(m));
            active &= ~m;
        }
        __syncthreads();
        for (uint32_t e2 = tid; e2 < num_experts; e2 += kGroupThreads) {
            const int32_t start = s_cur[e2];
            int32_t run = 0;
            for (int w = 0; w < kGroupWaves; ++w) {
                const int32_t c = s_tbl[w][e2];
                s_tbl[w][e2] = static_cast<uint16_t>(run);
                run += c;
            }
            s_base[e2] = start;
            s_cur[e2] = start + run;
        }
        __syncthreads();
        if (valid) order[s_base[e] + s_tbl[wave][e] + rank] = static_cast<int32_t>(p);
        __syncthreads();  // (the table is cleared again in the next round)
    }
}

constexpr int kMoeWaves = 4;
constexpr int kMoeCols = 4;  // routed tokens of one expert handled per pass over its rows

__device__ __forceinline__ float silu(float v) { return v * (1.0f / (1.0f + expf(-v))); }

// grid (ceil(inter / kMoeWaves), E).  Each wave owns gate row i and up row inter + i of
// expert e and produces h[pair, i] = silu(gate . x) * (up . x) for every pair routed to e.
__global__ __launch_bounds__(kMoeWaves * 64) void moe_gate_up_kernel(
    const uint8_t* __restrict__ gate_up, uint32_t inter, uint32_t hidden,
    const float* __restrict__ x, uint32_t top_k, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ order, float* __restrict__ h) {
    const uint32_t e = blockIdx.y;
    const int32_t beg = offsets[e], end = offsets[e + 1];
    if (beg == end) return;
    const int lane = threadIdx.x & 63;
    const uint32_t i = blockIdx.x * kMoeWaves + (threadIdx.x >> 6);
    if (i >= inter) return;
    const uint32_t nb = hidden / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint8_t* base = gate_up + static_cast<size_t>(e) * 2 * inter * row_bytes;
    const uint8_t* rowp[2] = {base + static_cast<size_t>(i) * row_bytes,
                              base + static_cast<size_t>(inter + i) * row_bytes};
    for (int32_t c0 = beg; c0 < end; c0 += kMoeCols) {
        const float* xrow[kMoeCols];
        int32_t pair[kMoeCols];
#pragma unroll
        for (int b = 0; b < kMoeCols; ++b) {
            pair[b] = order[c0 + b < end ? c0 + b : beg];
            xrow[b] = x + static_cast<size_t>(pair[b] / static_cast<int32_t>(top_k)) * hidden;
        }
        float acc[2][kMoeCols] = {};
        q4_rows_dot<2, kMoeCols>(rowp, nb, xrow, lane, acc);
#pragma unroll
        for (int b = 0; b < kMoeCols; ++b) {
            const float g = wave_sum(acc[0][b]);
            const float u = wave_sum(acc[1][b]);
            if (lane == 0 && c0 + b < end) h[static_cast<size_t>(pair[b]) * inter + i] = silu(g) * u;
        }
    }
}

// grid (ceil(hidden / (2*kMoeWaves)), E).  o[pair, r] = W_down[e][r, :] . h[pair, :].
__global__ __launch_bounds__(kMoeWaves * 64) void moe_down_kernel(
    const uint8_t* __restrict__ down, uint32_t inter, uint32_t hidden,
    const float* __restrict__ h, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ order, float* __restrict__ o) {
    const uint32_t e = blockIdx.y;
    const int32_t beg = offsets[e], end = offsets[e + 1];
    if (beg == end) return;
    const int lane = threadIdx.x & 63;
    const uint32_t r0 = (blockIdx.x * kMoeWaves + (threadIdx.x >> 6)) * 2;
    if (r0 >= hidden) return;
    const uint32_t nb = inter / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint8_t* base = down + static_cast<size_t>(e) * hidden * row_bytes;
    const uint32_t r1 = r0 + 1 < hidden ? r0 + 1 : r0;
    const uint8_t* rowp[2] = {base + static_cast<size_t>(r0) * row_bytes,
                              base + static_cast<size_t>(r1) * row_bytes};
    for (int32_t c0 = beg; c0 < end; c0 += kMoeCols) {
        const float* xrow[kMoeCols];
        int32_t pair[kMoeCols];
#pragma unroll
        for (int b = 0; b < kMoeCols; ++b) {
            pair[b] = order[c0 + b < end ? c0 + b : beg];
            xrow[b] = h + static_cast<size_t>(pair[b]) * inter;
        }
        float acc[2][kMoeCols] = {};
        q4_rows_dot<2, kMoeCols>(rowp, nb, xrow, lane, acc);
#pragma unroll
        for (int b = 0; b < kMoeCols; ++b) {
            const float v0 = wave_sum(acc[0][b]);
            const float v1 = wave_sum(acc[1][b]);
            if (lane == 0 && c0 + b < end) {
                o[static_cast<size_t>(pair[b]) * hidden + r0] = v0;
                if (r0 + 1 < hidden) o[static_cast<size_t>(pair[b]) * hidden + r0 + 1] = v1;
            }
        }
    }
}

// y[t, c] = sum over slots, in slot order, of weights[t, s] * o[t*top_k + s, c].
// R slots at a time: their routing entries, then their rows, are loaded together (the launcher picks R so that
// the usual slot counts are one round without padding: a padded slot is a row load for nothing).
template <int R>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ o,
                                                          const int32_t* __restrict__ ids,
                                                          const float* __restrict__ weights,
                                                          uint32_t num_experts, uint32_t top_k,
                                                          uint32_t hidden, float* __restrict__ y) {
    const uint32_t t = blockIdx.y;
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= hidden) return;
    float acc = 0.0f;
    for (uint32_t s0 = 0; s0 < top_k; s0 += R) {
        float wv[R], ov[R];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const uint32_t s = s0 + i < top_k ? s0 + i : top_k - 1;
            const int32_t e = ids[t * top_k + s];
            const bool ok = s0 + i < top_k && e >= 0 && e < static_cast<int32_t>(num_experts);
            wv[i] = ok ? weights[t * top_k + s] : 0.0f;
            ov[i] = o[static_cast<size_t>(t * top_k + s) * hidden + c];
            if (!ok) ov[i] = 0.0f;  // rows of invalid slots are never written
        }
#pragma unroll
        for (int i = 0; i < R; ++i) acc += wv[i] * ov[i];
    }
    y[static_cast<size_t>(t) * hidden + c] = acc;
}

template <int R>
void launch_combine_r(const float* o, const int32_t* ids, const float* weights, uint32_t experts, uint32_t slots,
                      uint32_t hidden, uint32_t tokens, float* y, hipStream_t stream) {
    hipLaunchKernelGGL(moe_combine_kernel<R>, dim3((hidden + 255) / 256, tokens), dim3(256), 0, stream, o, ids, weights,
                       experts, slots, hidden, y);
}

void launch_combine(const float* o, const int32_t* ids, const float* weights, uint32_t experts, uint32_t slots,
                    uint32_t hidden, uint32_t tokens, float* y, hipStream_t stream) {
    // (adding a padded product of zeros changes no bit of the sum, so R is free to choose)
    if (slots <= 2) launch_combine_r<2>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
    else if (slots <= 4) launch_combine_r<4>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
    else if (slots == 9) launch_combine_r<9>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
    else if (slots > 8 && slots <= 12) launch_combine_r<12>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
    else if (slots == 17) launch_combine_r<17>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
    else launch_combine_r<8>(o, ids, weights, experts, slots, hidden, tokens, y, stream);
}

}  // namespace

void launch_moe_route(const float* logits, uint32_t tokens, uint32_t num_experts, uint32_t top_k,
                      int32_t* ids, float* weights, hipStream_t stream, const float* x, const float* shared_gate,
                      uint32_t hidden) {
    const uint32_t out_stride = shared_gate ? top_k + 1 : top_k;
    if (num_experts <= 256)
        hipLaunchKernelGGL(moe_route_kernel<4>, dim3(tokens), dim3(64), 0, stream, logits, tokens, num_experts, top_k,
                           ids, weights, out_stride, x, shared_gate, hidden);
    else
        hipLaunchKernelGGL(moe_route_kernel<kMaxExperts / 64>, dim3(tokens), dim3(64), 0, stream, logits, tokens,
                           num_experts, top_k, ids, weights, out_stride, x, shared_gate, hidden);
}

void launch_moe_grouped(const uint8_t* gate_up, const uint8_t* down, uint32_t num_experts,
                        uint32_t inter, uint32_t hidden, const float* x, uint32_t tokens,
                        const int32_t* ids, const float* weights, uint32_t top_k, float* y,
                        const MoeScratch& s, hipStream_t stream, const uint8_t* shared_gate_up,
                        const uint8_t* shared_down) {
    // A shared expert rides along as expert `num_experts` in slot `top_k` of every token (the routing table then
    // has top_k + 1 slots per token): every kernel below simply sees one more expert and one more slot.
    const bool shared = shared_gate_up != nullptr;
    const uint32_t experts = num_experts + (shared ? 1 : 0), slots = top_k + (shared ? 1 : 0);
    const uint32_t pairs = tokens * slots;
    // matrix-core kernels whenever one pass's activations fit in LDS; the plain kernels otherwise
    const bool mfma_up = moe_i8_serves(hidden), mfma_down = moe_i8_serves(inter);
    // Up to 512 pairs the expert kernels read the routing table themselves (a thread per pair): no grouping launch, no
    // offsets -> order -> row chain of dependent loads, and they enumerate the (expert, pass) combinations that
    // exist, so the grid has no workgroups for the others.
    const bool scan = mfma_up && mfma_down && pairs <= kMoeIdsMaxPairs && experts <= kMoeIdsMaxExperts;
    const int32_t* scan_ids = scan ? ids : nullptr;
    if (!scan)
        hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(kGroupThreads), 0, stream, ids, pairs, experts, s.counts,
                           s.offsets, s.order);
    if (mfma_up)
        launch_moe_gate_up_i8(gate_up, experts, inter, hidden, x, tokens, slots, s.offsets, s.order, scan_ids,
                                s.h, stream, shared_gate_up);
    else
        hipLaunchKernelGGL(moe_gate_up_kernel, dim3((inter + kMoeWaves - 1) / kMoeWaves, num_experts),
                           dim3(kMoeWaves * 64), 0, stream, gate_up, inter, hidden, x, top_k, s.offsets,
                           s.order, s.h);
    if (mfma_down)
        launch_moe_down_i8(down, experts, inter, hidden, s.h, tokens, slots, s.offsets, s.order, scan_ids, s.o,
                             stream, shared_down);
    else
        hipLaunchKernelGGL(moe_down_kernel, dim3((hidden + 2 * kMoeWaves - 1) / (2 * kMoeWaves), num_experts),
                           dim3(kMoeWaves * 64), 0, stream, down, inter, hidden, s.h, s.offsets, s.order,
                           s.o);
    launch_combine(s.o, ids, weights, experts, slots, hidden, tokens, y, stream);
}

}  // namespace lq4
