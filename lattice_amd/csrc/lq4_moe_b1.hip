// Routed experts for a few tokens (decode): every (token, slot) pair is served as a one-token GEMV in
// the arithmetic of the batch-1 kernel (lq4_b1_dev.hpp: 4-bit dot products on packed dwords, fixed-point
// activations scaled per block), two launches for the whole step:
//   1. gate||up: for token t the selected experts' [2I, H] matrices are one virtual matrix of
//      top_k * 2I rows over x[t], walked in (gate row, up row) pairs: pair q belongs to slot q / I and
//      reads rows q % I and I + q % I of expert ids[t, slot].  A wave meets the two rows of a pair one
//      after the other and writes act[t, q] = silu(g) * u * w_slot, so neither g nor u reaches memory.
//   2. down: y[t] = sum_s W_down[e_s] . act[t, s] is ONE GEMV over a K of top_k * I: block b of a row
//      belongs to slot b / (I/32) and is read from that expert's matrix.  The weighted sum over the
//      slots happens inside the dot product, so there is no combine launch.
// accumulate_routed_experts (crates/inference/src/model/qwen35/moe.rs:127-190) visits a token's
// selected experts one after the other; with one token no two pairs share an expert, so nothing is
// read twice, and with a few tokens the little that is costs less than the grouped kernels' fixed
// parts (lq4_moe_i8.hip serves larger steps, where tokens do share experts).
// Slots with an id outside [0, E) are skipped as the reference skips them (moe.rs:147-149): they read
// expert 0 (any valid address) and enter the sum with weight 0.
// The shared expert (moe.rs:194-250) can ride along as one more slot with the weight
// sigmoid(x . shared_gate): its 2 MB then cost two slightly longer launches instead of three more.
// The router (moe.rs:39-125) can run inside the gate||up launch as well: one wave of every workgroup
// repeats it for the workgroup's token (64 logits, eight wave-wide maxima), which costs each workgroup
// about a microsecond before its first weight request and saves a launch of four.
#include "lq4_b1_dev.hpp"
#include "lq4_moe_route_dev.hpp"

namespace lq4 {

namespace {

using namespace b1;

struct MoeB1Args {
    const uint8_t* w;     // gate||up [E, 2I, H] or down [E, H, I], native blocks
    const float* x;       // gate||up: x [tokens, H];  down: act [tokens, slots * I]
    float* y;             // gate||up: act;  down: y [tokens, H]
    const int32_t* ids;   // [tokens, top_k]
    const float* wts;     // [tokens, top_k]
    uint32_t num_experts, top_k, inter, hidden;
    uint32_t n, k;        // rows and reduction length of the virtual matrix of one token
    // The always-active shared expert (apply_shared_expert, moe.rs:194-250) as one more slot behind the
    // routed ones, when its intermediate size equals the routed experts': its own tensors (`w_shared`,
    // the gate||up or the down one), and as its weight sigmoid(x . shared_gate), which workgroup 0 of the
    // gate||up launch computes into shared_wt[token] for the down launch (which applies it while it stages:
    // the gate||up launch writes that slot's act without a weight).  slots = top_k (+ 1).
    const uint8_t* w_shared;
    const float* shared_gate;
    float* shared_wt;
    uint32_t slots;
    // gate||up launch only: route inside the launch.  Wave 0 of every workgroup runs the router of its token
    // from route_logits [tokens, E] (E <= 256) and the workgroup takes the ids from LDS; workgroup 0 of each
    // token also stores ids and weights to ids_out / wts_out, where the down launch reads them.
    const float* route_logits;
    int32_t* ids_out;
    float* wts_out;
    uint32_t accumulate;  // down launch: y += the result instead of y = (the shared expert alone, onto the routed sum)
};

__device__ __forceinline__ float silu_mul(float gate, float u) {
    // hardware exp2 and reciprocal (about 1 ulp each), as the fused one-token GEMV evaluates it
    const float e = __builtin_amdgcn_exp2f(gate * -1.44269504088896340736f);
    return gate * __builtin_amdgcn_rcpf(1.0f + e) * u;
}

// grid (workgroups per token, tokens), block 256.  Wave `wid` of a token's `n_waves` works through
// chunks of RW rows; the next chunk's blocks are in flight while the current one is consumed.  Down: row
// i * n_waves + wid is the wave's i-th.  Gate||up: its i-th row is the gate (i even) or up (i odd) row of
// pair (i / 2) * n_waves + wid.  SLABS = ceil(K / 2048): a lane owns block slab * 64 + lane
// of a row.  Dynamic LDS: (K / 32) * kXPitch dwords.
// ROUTE (gate||up only): the router runs inside the launch (a separate instantiation, so that the plain one
// carries none of it).
template <bool DOWN, int RW, int SLABS, bool ROUTE>
__global__ __launch_bounds__(256) void moe_b1_kernel(MoeB1Args a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t xs[];
    lds_u32* const xsl = (lds_u32*)xs;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t token = blockIdx.y;
    const uint32_t nb = a.k / kBlockWeights;
    const uint32_t nbe = a.inter / kBlockWeights;  // blocks of one expert's down row
    const int32_t* ids = a.ids + static_cast<size_t>(token) * a.top_k;
    const float* wts = a.wts + static_cast<size_t>(token) * a.top_k;
    __shared__ int32_t s_ids[ROUTE ? 16 : 1];
    __shared__ float s_wts[ROUTE ? 16 : 1];
    auto expert_of = [&](uint32_t slot) {  // the shared expert's tensor holds one expert
        const int32_t e = slot < a.top_k ? (ROUTE ? s_ids[slot] : ids[slot]) : 0;
        return (e >= 0 && static_cast<uint32_t>(e) < a.num_experts) ? static_cast<uint32_t>(e) : 0u;
    };
    // Read here, under a condition that is the same for the whole launch: inside weight_of the load would
    // sit behind a per-lane condition, where the compiler turns it into a scalar load that every wave
    // executes whatever its lanes decided, i.e. also through the null pointer of a launch without a
    // shared expert.
    float shared_w = 0.0f;
    if (DOWN && a.shared_wt != nullptr) shared_w = a.shared_wt[token];
    // Routing weight of a slot (`slot` is the same for the whole wave wherever this is called); a slot with an
    // id outside [0, E) counts 0.  The shared expert's slot: 1 in the gate||up launch, its weight in the down one.
    auto weight_of = [&](uint32_t slot) {
        if (slot >= a.top_k) return DOWN ? shared_w : 1.0f;
        const int32_t e = ROUTE ? s_ids[slot] : ids[slot];
        const float w = ROUTE ? s_wts[slot] : wts[slot];
        return (e >= 0 && static_cast<uint32_t>(e) < a.num_experts) ? w : 0.0f;
    };
    auto tensor_of = [&](uint32_t slot) { return slot < a.top_k ? a.w : a.w_shared; };

    // ---- activations first: their loads are waited for alone, ahead of the weights ----
    constexpr int kUnitsPerThread = 4;  // K <= 8192: 1024 units of 8 activations
    const uint32_t n_units = nb * 4;
    float4 va[kUnitsPerThread], vb[kUnitsPerThread];
    float wt[kUnitsPerThread];
#pragma unroll
    for (int i = 0; i < kUnitsPerThread; ++i) {
        const uint32_t g = tid + i * 256 < n_units ? tid + i * 256 : 0;
        const uint32_t blk = g >> 2, dw = g & 3;
        if constexpr (!DOWN) {
            const float4* xp = reinterpret_cast<const float4*>(a.x + static_cast<size_t>(token) * a.hidden + blk * kBlockWeights + dw * 8);
            va[i] = xp[0];
            vb[i] = xp[1];
            wt[i] = 1.0f;
        } else {
            const float* hp = a.x + static_cast<size_t>(token) * a.k + blk * kBlockWeights + dw * 8;
            va[i] = reinterpret_cast<const float4*>(hp)[0];
            vb[i] = reinterpret_cast<const float4*>(hp)[1];
            wt[i] = blk / nbe >= a.top_k ? shared_w : 1.0f;  // the routed slots carry their weight already
        }
    }

    if constexpr (ROUTE) {
        {
            __shared__ float s_ev[256];
            if (tid < 64) {
                int32_t id;
                float w;
                route_one_token<4>(a.route_logits + static_cast<size_t>(token) * a.num_experts, a.num_experts, a.top_k, lane,
                                   s_ev, id, w);
                if (lane < a.top_k) {
                    s_ids[lane] = id;
                    s_wts[lane] = w;
                    if (blockIdx.x == 0) {
                        a.ids_out[static_cast<size_t>(token) * a.top_k + lane] = id;
                        a.wts_out[static_cast<size_t>(token) * a.top_k + lane] = w;
                    }
                }
            }
            __syncthreads();
        }
    }

    // ---- rows of this wave ----
    const uint32_t n_waves = gridDim.x * 4;
    const uint32_t wid = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (tid >> 6));
    const uint32_t items = DOWN ? a.n : a.n / 2;  // rows, or (gate, up) pairs
    const uint32_t mine = wid < items ? (items - wid + n_waves - 1) / n_waves : 0;
    const uint32_t chunks = ((DOWN ? mine : 2 * mine) + RW - 1) / RW;
    // where this lane's block of each slab lives, apart from the row
    uintptr_t lane_base[SLABS];  // DOWN: the slot's tensor and expert and the block; else only the block's offset
    bool live[SLABS];
#pragma unroll
    for (int t = 0; t < SLABS; ++t) {
        uint32_t blk = t * 64 + lane;
        live[t] = blk < nb;
        if (!live[t]) blk = nb - 1;
        if constexpr (DOWN) {
            const uint32_t slot = blk / nbe, kb = blk - slot * nbe;
            lane_base[t] = reinterpret_cast<uintptr_t>(tensor_of(slot)) +
                           (static_cast<size_t>(expert_of(slot)) * a.hidden * nbe + kb) * kBlockBytes;
        } else {
            lane_base[t] = static_cast<size_t>(blk) * kBlockBytes;
        }
    }
    auto load_chunk = [&](Q4BlockRaw (&buf)[RW][SLABS], uint32_t c) {
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const uint32_t i = c * RW + j;  // scalar, like everything derived from it
            uintptr_t row_off;  // the row's part of the address (with the tensor, for gate||up)
            if constexpr (DOWN) {
                uint32_t row = i * n_waves + wid;
                if (row >= a.n) row = a.n - 1;
                row_off = static_cast<size_t>(row) * nbe * kBlockBytes;
            } else {
                uint32_t q = (i >> 1) * n_waves + wid;
                if (q >= items) q = items - 1;
                const uint32_t slot = q / a.inter, r = (i & 1) * a.inter + (q - slot * a.inter);
                row_off = reinterpret_cast<uintptr_t>(tensor_of(slot)) +
                          (static_cast<size_t>(expert_of(slot)) * 2 * a.inter + r) * nb * kBlockBytes;
            }
#pragma unroll
            for (int t = 0; t < SLABS; ++t) {
                // (an address built from integers: say that it is global memory, or the loads become flat ones)
                const LQ4_GLOBAL uint8_t* bp = (const LQ4_GLOBAL uint8_t*)(lane_base[t] + row_off);
                buf[j][t].sb = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL uint32_t*>(bp));
                const u32x4u q = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL u32x4u*>(bp + 4));
                buf[j][t].q[0] = q.x; buf[j][t].q[1] = q.y; buf[j][t].q[2] = q.z; buf[j][t].q[3] = q.w;
            }
        }
    };
    Q4BlockRaw buf_a[RW][SLABS], buf_b[RW][SLABS];
    if (chunks) load_chunk(buf_a, 0);
    __builtin_amdgcn_sched_barrier(0);  // the weight loads stay behind the activation loads above

    // ---- stage ----
#pragma unroll
    for (int i = 0; i < kUnitsPerThread; ++i) {
        const uint32_t g = tid + i * 256;
        float4 p = va[i], q = vb[i];
        if constexpr (DOWN) {
            p.x *= wt[i]; p.y *= wt[i]; p.z *= wt[i]; p.w *= wt[i];
            q.x *= wt[i]; q.y *= wt[i]; q.z *= wt[i]; q.w *= wt[i];
        }
        // whole quads call together: a quad's four units are one block, all inside or all outside
        if (i * 256 < n_units) stage_x8(xsl, g < n_units ? g : 0, p, q, g < n_units);
    }
    barrier_lds();
    if constexpr (!DOWN) {
        // the shared expert's weight for the down launch: sigmoid(x . shared_gate), by one workgroup
        if (a.shared_wt && blockIdx.x == 0) {
            __shared__ float part[4];
            float dot = 0.0f;
#pragma unroll
            for (int i = 0; i < kUnitsPerThread; ++i) {
                const uint32_t g = tid + i * 256;
                if (g < n_units) {
                    const float4* gp = reinterpret_cast<const float4*>(a.shared_gate + (g >> 2) * kBlockWeights + (g & 3) * 8);
                    const float4 g0 = gp[0], g1 = gp[1];
                    dot = fmaf(va[i].x, g0.x, dot); dot = fmaf(va[i].y, g0.y, dot);
                    dot = fmaf(va[i].z, g0.z, dot); dot = fmaf(va[i].w, g0.w, dot);
                    dot = fmaf(vb[i].x, g1.x, dot); dot = fmaf(vb[i].y, g1.y, dot);
                    dot = fmaf(vb[i].z, g1.z, dot); dot = fmaf(vb[i].w, g1.w, dot);
                }
            }
            dot = segment_sum<64>(dot);
            if (lane == 63) part[tid >> 6] = dot;
            __syncthreads();
            if (tid == 0) a.shared_wt[token] = 1.0f / (1.0f + expf(-((part[0] + part[1]) + (part[2] + part[3]))));
        }
    }

    XBlock xb_[SLABS];
#pragma unroll
    for (int t = 0; t < SLABS; ++t) load_xblock(xsl, live[t] ? t * 64 + lane : nb - 1, xb_[t]);

    float gate_kept = 0.0f;  // gate||up: the gate row's sum until the pair's up row is done
    auto consume = [&](Q4BlockRaw (&cur)[RW][SLABS], uint32_t c) {
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            float acc = 0.0f;
#pragma unroll
            for (int t = 0; t < SLABS; ++t) acc = block_fma(cur[j][t], xb_[t], live[t], acc);
            acc = segment_sum<64>(acc);
            const uint32_t i = c * RW + j;
            if constexpr (DOWN) {
                const uint32_t row = i * n_waves + wid;
                if (lane == 63 && row < a.n) {
                    float* dst = a.y + static_cast<size_t>(token) * a.n + row;
                    *dst = a.accumulate ? *dst + acc : acc;
                }
            } else if ((i & 1) == 0) {
                gate_kept = acc;
            } else {
                const uint32_t q = (i >> 1) * n_waves + wid;
                if (q < items) {  // (the same for the whole wave)
                    const float w = weight_of(q / a.inter);
                    if (lane == 63) a.y[static_cast<size_t>(token) * items + q] = silu_mul(gate_kept, acc) * w;
                }
            }
        }
    };
    uint32_t c = 0;
    for (; c + 2 <= chunks; c += 2) {
        load_chunk(buf_b, c + 1);
        consume(buf_a, c);
        if (c + 2 < chunks) load_chunk(buf_a, c + 2);
        consume(buf_b, c + 1);
    }
    if (c < chunks) consume(buf_a, c);
}

template <bool DOWN, bool ROUTE = false>
void launch_one(const MoeB1Args& a, uint32_t tokens, hipStream_t stream) {
    const uint32_t nb = a.k / kBlockWeights;
    const uint32_t slabs = (nb + 63) / 64;
    const uint32_t rw = slabs == 1 ? 4 : slabs <= 3 ? 2 : 1;
    const size_t lds = static_cast<size_t>(nb) * kXPitch * 4;
    // all waves of the step resident at once where the rows allow: 4096 waves over the tokens
    // (gate||up with one row per chunk: a wave needs two chunks for a pair, so a wave per pair is the most)
    const uint32_t wave_rows = (!DOWN && rw == 1) ? a.n / 2 : (a.n + rw - 1) / rw;
    uint32_t budget = 4096 / tokens;
    if (budget < 64) budget = 64;
    const uint32_t waves = wave_rows < budget ? wave_rows : budget;
    const dim3 grid((waves + 3) / 4, tokens), block(256);
#define LQ4_MOE_B1(RW_, SL_)                                                                                   \
    do {                                                                                                       \
        static LdsCapOnce lds_cap;                                                                             \
        lds_cap.raise(reinterpret_cast<const void*>(moe_b1_kernel<DOWN, RW_, SL_, ROUTE>), 64 * 1024);         \
        hipLaunchKernelGGL((moe_b1_kernel<DOWN, RW_, SL_, ROUTE>), grid, block, lds, stream, a);               \
    } while (0)
    if (slabs == 1) LQ4_MOE_B1(4, 1);
    else if (slabs == 2) LQ4_MOE_B1(2, 2);
    else if (slabs == 3) LQ4_MOE_B1(2, 3);
    else LQ4_MOE_B1(1, 4);
#undef LQ4_MOE_B1
}

}  // namespace

bool moe_b1_serves(uint32_t inter, uint32_t hidden, uint32_t slots) {
    const uint64_t k_down = static_cast<uint64_t>(slots) * inter;
    return hidden % kBlockWeights == 0 && inter % kBlockWeights == 0 && hidden <= 8192 && k_down <= 8192;
}

size_t moe_b1_scratch_bytes(uint32_t tokens, uint32_t slots, uint32_t inter) {
    // act [tokens, slots * I], then the shared expert's weight per token
    return static_cast<size_t>(tokens) * slots * inter * sizeof(float) + static_cast<size_t>(tokens) * sizeof(float);
}

void launch_moe_b1(const uint8_t* gate_up, const uint8_t* down, uint32_t num_experts, uint32_t inter, uint32_t hidden,
                   const float* x, uint32_t tokens, const int32_t* ids, const float* weights, uint32_t top_k, float* y,
                   float* scratch, const uint8_t* shared_gate_up, const uint8_t* shared_down, const float* shared_gate,
                   const float* route_logits, int32_t* ids_out, float* wts_out, bool accumulate, hipStream_t stream) {
    const uint32_t slots = shared_gate_up ? top_k + 1 : top_k;
    float* h = scratch;
    float* shared_wt = shared_gate_up ? scratch + static_cast<size_t>(tokens) * slots * inter : nullptr;
    if (route_logits) {  // the gate||up launch routes; the down launch reads what it stored
        ids = ids_out;
        weights = wts_out;
    }
    MoeB1Args g{gate_up, x, h, ids, weights, num_experts, top_k, inter, hidden, slots * 2 * inter, hidden,
                shared_gate_up, shared_gate, shared_wt, slots, route_logits, ids_out, wts_out, 0u};
    if (route_logits) launch_one<false, true>(g, tokens, stream);
    else launch_one<false>(g, tokens, stream);
    MoeB1Args d{down, h, y, ids, weights, num_experts, top_k, inter, hidden, hidden, slots * inter,
                shared_down, shared_gate, shared_wt, slots, nullptr, nullptr, nullptr, accumulate ? 1u : 0u};
    launch_one<true>(d, tokens, stream);
}

}  // namespace lq4
