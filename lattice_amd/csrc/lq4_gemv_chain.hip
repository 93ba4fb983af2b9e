// A chain of dependent batch-1 GEMVs in ONE launch: the device twin of the reference encoding a whole
// token into one command buffer (forward/metal_qwen35.rs:6943 forward_step, commit at :6447;
// encode_mlp_block in inner/layers/mod.rs; the elementwise dispatches at inner/dispatch.rs:916-930,
// 1171-1290).  Step j is y_j = W_j . x_j with x_j either an external vector or the previous step's
// result, passed through the same prologues/epilogues as the fused batch-1 GEMV:
//   o -> (+residual) -> RMSNorm -> gate||up -> silu*up -> down -> (+residual) -> RMSNorm -> qkv ...
//
// Why one launch.  A 3-16 MB GEMV is over in 2-3 us, of which launch ramp, the first HBM round trip
// and the drain are most; four launches pay that four times and the memory pipe runs dry between
// them.  Here the grid is resident for the whole chain (one workgroup per CU) and every wave asks
// for the weights of step j+1 and j+2 before step j's result exists: weights do not depend on
// activations, only the order of the arithmetic does.
//
// Work layout per step.  As in the batch-1 kernel a lane owns whole 20-byte blocks: lane l of a wave
// reads block 64*s + l of a row (slab s), so a wave's load pair covers 1280 contiguous bytes.  A
// wave takes row groups g = wave, wave + W, ... (W = waves in the grid); a group is one row, or the
// pair (g, g + N/2) when the step ends in silu(gate) * up.  All of a wave's blocks of a step sit in
// kChainSlots register slots, so steps of up to kChainSlots * 64 * W blocks (25 M weights on 256 CUs)
// are eligible; larger ones are run by the per-step fallback in the C ABI layer.
//
// Hand-over.  The result vector of step j goes to library scratch as 64-bit words
// {f32 value, launch epoch}, one agent-scope (L2-coherent across the XCDs) relaxed atomic store per
// row; value and tag travel together, so a reader needs no fence and no separate flag: it polls its
// slice of the vector with agent-scope atomic loads until every word carries this launch's epoch.
// These loads hit in the reader's own L2 until a writer's store invalidates the line (~110 ns a
// poll, ~0.6-0.8 us from store to sight across XCDs, measured).  The epoch is a word in the context:
// every workgroup reads it when it starts, workgroup 0 advances it when it has finished, which is
// after every workgroup has read it as soon as the chain has one dependent step.  Nothing is reset
// between launches, so a captured launch can be replayed.  The wait is bounded (spin_limit polls):
// a wave that runs out raises the context's failure word and its workgroup leaves; the others run
// out the same way, so every kernel exits and lq4_sync reports the failure.
#include "lq4_b1_dev.hpp"

namespace lq4 {

namespace {

using namespace b1;

constexpr int kChainWaves = 8;
constexpr int kChainThreads = kChainWaves * 64;
constexpr int kChainSlots = 6;  // blocks per lane and step
constexpr int kChainUnits = 4;  // 8-activation units per thread and step: K <= 4 * 8 * 512 = 16384

__device__ __forceinline__ unsigned long long tag_word(float v, uint32_t epoch) {
    return (static_cast<unsigned long long>(epoch) << 32) | __builtin_bit_cast(uint32_t, v);
}

constexpr uint32_t kStepDwords = sizeof(ChainStep) / 4;
static_assert(sizeof(ChainStep) == 128, "the descriptor copy assumes 32 dwords a step");

// Step j's descriptor out of LDS, every field uniform again (scalar registers).
__device__ __forceinline__ ChainStep read_step(const lds_u32* desc, uint32_t j) {
    uint32_t raw[kStepDwords];
    const LQ4_LDS u32x4* p = reinterpret_cast<const LQ4_LDS u32x4*>(desc + j * kStepDwords);
#pragma unroll
    for (uint32_t i = 0; i < kStepDwords / 4; ++i) {
        const u32x4 v = p[i];
        raw[4 * i + 0] = v.x; raw[4 * i + 1] = v.y; raw[4 * i + 2] = v.z; raw[4 * i + 3] = v.w;
    }
#pragma unroll
    for (uint32_t i = 0; i < kStepDwords; ++i) raw[i] = __builtin_amdgcn_readfirstlane(raw[i]);
    ChainStep st;
    __builtin_memcpy(&st, raw, sizeof st);
    return st;
}

__device__ __forceinline__ float silu_mul_fast(float gate, float up) {
    // hardware exp2 and reciprocal (about 1 ulp each), as the fused batch-1 prologue
    const float e = __builtin_amdgcn_exp2f(gate * -1.44269504088896340736f);
    return gate * __builtin_amdgcn_rcpf(1.0f + e) * up;
}

__device__ __forceinline__ void ld8(const float* p, float (&o)[8]) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const LQ4_GLOBAL f32x4* q = reinterpret_cast<const LQ4_GLOBAL f32x4*>(as_global(p));
    const f32x4 lo = q[0], hi = q[1];
    o[0] = lo.x; o[1] = lo.y; o[2] = lo.z; o[3] = lo.w;
    o[4] = hi.x; o[5] = hi.y; o[6] = hi.z; o[7] = hi.w;
}

// Dynamic LDS: two activation buffers of xs_dwords each (steps alternate), kChainWaves floats for the
// sum of squares, the abort word, then the step descriptors.
__global__ __launch_bounds__(kChainThreads) void gemv_chain_kernel(const ChainArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint32_t lds_raw[];
    lds_u32* const lds = (lds_u32*)lds_raw;
    constexpr int T = kChainThreads;
    const int tid = threadIdx.x, lane = tid & 63;
    LQ4_LDS float* const red = reinterpret_cast<LQ4_LDS float*>(lds + 2 * a.xs_dwords);
    lds_u32* const abort_flag = lds + 2 * a.xs_dwords + kChainWaves;
    lds_u32* const desc = lds + 2 * a.xs_dwords + kChainWaves + 4;  // 16-byte aligned
    const uint32_t n_waves = gridDim.x * kChainWaves;
    const uint32_t wid = __builtin_amdgcn_readfirstlane(blockIdx.x * kChainWaves + (tid >> 6));
    if (tid == 0) *abort_flag = 0;
    // The step descriptors are kernel arguments.  Read with scalar loads where they are needed, the
    // first touch of each of their cache lines would sit on the critical path of its step.  One
    // vector load per thread copies all of them to LDS now; the steps read them from there (same
    // address in every lane) and make them scalar again.
    {
        const uint32_t* ka = reinterpret_cast<const uint32_t*>(&a.s[0]);
        if (static_cast<uint32_t>(tid) < a.n_steps * kStepDwords) desc[tid] = ka[tid];
        static_assert(kMaxChainSteps * kStepDwords <= kChainThreads, "one descriptor dword per thread");
    }
    const uint32_t epoch = *as_global(a.epoch);
#ifdef LQ4_CHAIN_TRACE
    uint32_t trace_at = 0;
    auto mark = [&]() {
        if (lane == 0 && a.trace) as_global(a.trace)[static_cast<size_t>(wid) * 32 + trace_at] = wall_clock64();
        ++trace_at;
    };
#else
    auto mark = []() {};
#endif
    mark();
    __syncthreads();

    // ---- weights (and residual inputs) of a whole step into one register set ----
    // Always the same number of loads, none behind a condition: the compiler's wait counts are then
    // exact, and a later step's loads can stay in flight while an earlier step's registers are used.
    auto load_step = [&](Q4BlockRaw (&buf)[kChainSlots], float (&res)[kChainSlots], uint32_t j) {
        // (a step past the end of the chain is requested as well, as re-reads of step 0's first rows
        // that every wave shares: a prefetch behind a condition would make the compiler wait for the
        // newest loads before it lets the current step's registers be used)
        const bool past_end = j >= a.n_steps;
        ChainStep st = read_step(desc, past_end ? 0 : j);
        if (past_end) st.groups = 0;
        const uint32_t nb = st.k / kBlockWeights;
        const uint32_t row_bytes = nb * kBlockBytes;
        const uint32_t g0 = wid < st.groups ? wid : 0;  // slots without work re-read a block of this one
        // residual input: a plain float vector, the value words of an earlier tagged result, or (no
        // residual) any readable word
        const uint32_t* res_base = st.res_tagged ? reinterpret_cast<const uint32_t*>(st.res_tagged)
                                   : st.res_plain ? reinterpret_cast<const uint32_t*>(st.res_plain)
                                                  : reinterpret_cast<const uint32_t*>(st.w);
        const uint32_t res_stride = st.res_tagged ? 2 : st.res_plain ? 1 : 0;
        uint32_t g = wid, rsel = 0, slab = 0;
#pragma unroll
        for (int s = 0; s < kChainSlots; ++s) {
            const uint32_t gg = g < st.groups ? g : g0;
            const uint32_t row = gg + (rsel ? st.n / 2 : 0);
            uint32_t blk = slab * 64 + lane;
            if (blk >= nb) blk = nb - 1;
            const LQ4_GLOBAL uint8_t* p = as_global(st.w) + static_cast<size_t>(row) * row_bytes + blk * static_cast<uint32_t>(kBlockBytes);
            buf[s].sb = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL uint32_t*>(p));
            const u32x4u q = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL u32x4u*>(p + 4));
            buf[s].q[0] = q.x; buf[s].q[1] = q.y; buf[s].q[2] = q.z; buf[s].q[3] = q.w;
            res[s] = __builtin_bit_cast(float, __hip_atomic_load(as_global(res_base) + static_cast<size_t>(row) * res_stride,
                                                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            if (++slab == st.slabs) {
                slab = 0;
                if (++rsel == st.group_rows) {
                    rsel = 0;
                    g += n_waves;
                }
            }
        }
    };

    // ---- one step's arithmetic out of a register set, with its epilogue and the tagged store ----
    auto compute_step = [&](const Q4BlockRaw (&buf)[kChainSlots], const float (&res)[kChainSlots], uint32_t j,
                            const lds_u32* xs) {
        const ChainStep st = read_step(desc, j);
        const uint32_t nb = st.k / kBlockWeights;
        uint32_t g = wid, rsel = 0, slab = 0, have_slab = 0xffffffffu;
        XBlock xb;
        float acc = 0.0f, v_gate = 0.0f;
#pragma unroll
        for (int s = 0; s < kChainSlots; ++s) {
            if (g < st.groups) {  // uniform across the wave
                const uint32_t blk_raw = slab * 64 + lane;
                const bool live = blk_raw < nb;
                if (slab != have_slab) {
                    load_xblock(xs, live ? blk_raw : nb - 1, xb);
                    have_slab = slab;
                }
                acc = block_fma(buf[s], xb, live, acc);
                if (slab + 1 == st.slabs) {  // row complete
                    float v = segment_sum<64>(acc);
                    acc = 0.0f;
                    uint32_t row_out = g + (rsel ? st.n / 2 : 0);
                    bool emit = true;
                    if (st.epilogue == ChainStep::kAddResidual) {
                        v += res[s];
                    } else if (st.epilogue == ChainStep::kSiluMulPairs) {
                        if (rsel == 0) {
                            v_gate = v;
                            emit = false;
                        } else {
                            v = silu_mul_fast(v_gate, v);
                            row_out = g;
                        }
                    }
                    if (emit && lane == 63) {
                        if (st.out_tagged)
                            __hip_atomic_store(as_global(st.out_tagged) + row_out, tag_word(v, epoch), __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
                        if (st.y) as_global(st.y)[row_out] = v;
                        if (st.res_out) as_global(st.res_out)[row_out] = v;
                    }
                }
            }
            if (++slab == st.slabs) {
                slab = 0;
                if (++rsel == st.group_rows) {
                    rsel = 0;
                    g += n_waves;
                }
            }
        }
    };

    // ---- the activations of step j: fetch (external loads, or polling the previous result) ----
    // v: the vector (x, base + delta, the previous result, or gate); aux: gamma or up.
    auto unit_at = [](uint32_t u) { return (u >> 2) * kBlockWeights + (u & 3) * 8; };
    auto fetch_x = [&](uint32_t j, float (&v)[kChainUnits][8], float (&aux)[kChainUnits][8]) {
        const ChainStep st = read_step(desc, j);
        const uint32_t n_units = st.k / 8;
        // gamma / up first: they depend on nothing
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
                const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
                if (st.prologue == ChainStep::kAddNorm) ld8(st.gamma + unit_at(u), aux[i]);
                else if (st.prologue == ChainStep::kSiluMul) ld8(st.x + st.k + unit_at(u), aux[i]);
            }
        }
        if (!st.x_tagged) {  // external activations
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i) {
                if (static_cast<uint32_t>(i * T) < n_units) {
                    const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
                    if (st.prologue == ChainStep::kAddNorm) {
                        ld8(st.base + unit_at(u), v[i]);
                        if (st.delta) {
                            float d[8];
                            ld8(st.delta + unit_at(u), d);
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[i][e] += d[e];
                        }
                    } else {
                        ld8(st.x + unit_at(u), v[i]);
                    }
                }
            }
            return;
        }
        // the previous step's result: poll this wave's slice until every word carries the epoch
        uint32_t spins = 0;
        while (true) {
            if (a.spin_limit == 0) {  // hand-over switched off: leave as a wave whose wait ran out does
                if (lane == 0) {
                    *abort_flag = 1;
                    __hip_atomic_store(as_global(a.fail), j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                break;
            }
            bool ok = true;
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i) {
                if (static_cast<uint32_t>(i * T) < n_units) {
                    const bool act = tid + i * T < n_units;
                    const LQ4_GLOBAL unsigned long long* p = as_global(st.x_tagged) + static_cast<size_t>(act ? tid + i * T : 0) * 8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const unsigned long long w = __hip_atomic_load(p + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        v[i][e] = __builtin_bit_cast(float, static_cast<uint32_t>(w));
                        ok = ok && (!act || static_cast<uint32_t>(w >> 32) == epoch);
                    }
                }
            }
            if (__all(ok)) break;
            if (++spins >= a.spin_limit) {
                if (lane == 0) {
                    *abort_flag = 1;
                    __hip_atomic_store(as_global(a.fail), j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
    };

    // ---- prologue arithmetic, conversion and the LDS store; ends with the step's barrier ----
    auto finish_x = [&](uint32_t j, float (&v)[kChainUnits][8], const float (&aux)[kChainUnits][8], lds_u32* xs) {
        const ChainStep st = read_step(desc, j);
        const uint32_t n_units = st.k / 8;
        if (st.prologue == ChainStep::kAddNorm) {
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i) {
                if (static_cast<uint32_t>(i * T) < n_units && tid + i * T < n_units) {
                    ss += ((v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3])) +
                          ((v[i][4] * v[i][4] + v[i][5] * v[i][5]) + (v[i][6] * v[i][6] + v[i][7] * v[i][7]));
                    if (blockIdx.x == 0 && st.residual_out) {
                        typedef float f32x4 __attribute__((ext_vector_type(4)));
                        LQ4_GLOBAL f32x4* rp = reinterpret_cast<LQ4_GLOBAL f32x4*>(as_global(st.residual_out) + unit_at(tid + i * T));
                        rp[0] = f32x4{v[i][0], v[i][1], v[i][2], v[i][3]};
                        rp[1] = f32x4{v[i][4], v[i][5], v[i][6], v[i][7]};
                    }
                }
            }
            ss = wave_sum(ss);
            if (lane == 0) red[tid >> 6] = ss;
            barrier_lds();
            const float total = ((red[0] + red[1]) + (red[2] + red[3])) + ((red[4] + red[5]) + (red[6] + red[7]));
            static_assert(kChainWaves == 8, "the sum of squares is combined for eight waves");
            const float inv_rms = 1.0f / sqrtf(total / static_cast<float>(st.k) + st.eps);
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i)
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * inv_rms * (1.0f + aux[i][e]);
        } else if (st.prologue == ChainStep::kSiluMul) {
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i)
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = silu_mul_fast(v[i][e], aux[i][e]);
        }
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
                const bool act = tid + i * T < n_units;
                stage_x8(xs, act ? tid + i * T : 0, make_float4(v[i][0], v[i][1], v[i][2], v[i][3]),
                         make_float4(v[i][4], v[i][5], v[i][6], v[i][7]), act);
            }
        }
        barrier_lds();
        return *abort_flag == 0;
    };

    Q4BlockRaw buf_a[kChainSlots], buf_b[kChainSlots];
    float res_a[kChainSlots], res_b[kChainSlots];
    float xv[kChainUnits][8], xaux[kChainUnits][8];
    lds_u32* const xs0 = lds;
    lds_u32* const xs1 = lds + a.xs_dwords;

    // the first activations are requested before any weight: loads return in order
    fetch_x(0, xv, xaux);
    load_step(buf_a, res_a, 0);
    load_step(buf_b, res_b, 1);
    mark();
    if (!finish_x(0, xv, xaux, xs0)) return;
    mark();

    // After step j's arithmetic its register set is free: it takes step j+2's weights once the
    // activations of step j+1 have been sighted (a poll issued behind a fresh burst of weight loads
    // would only return with the last of them).
    for (uint32_t j = 0; j < a.n_steps; j += 2) {
        compute_step(buf_a, res_a, j, xs0);
        mark();
        if (j + 1 >= a.n_steps) break;
        fetch_x(j + 1, xv, xaux);
        mark();
        load_step(buf_a, res_a, j + 2);
        if (!finish_x(j + 1, xv, xaux, xs1)) return;
        mark();
        compute_step(buf_b, res_b, j + 1, xs1);
        mark();
        if (j + 2 >= a.n_steps) break;
        fetch_x(j + 2, xv, xaux);
        mark();
        load_step(buf_b, res_b, j + 3);
        if (!finish_x(j + 2, xv, xaux, xs0)) return;
        mark();
    }
    // every workgroup read the epoch before workgroup 0 could get here through a dependent step
    if (blockIdx.x == 0 && tid == 0)
        __hip_atomic_store(as_global(a.epoch), epoch + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

size_t gemv_chain_lds_bytes(uint32_t k_max) {
    // two activation buffers | sums of squares | abort word | step descriptors (keeps 16-byte alignment:
    // the buffers are multiples of 144 bytes, 8 + 1 dwords follow, so pad to a multiple of 4 dwords)
    return (2 * static_cast<size_t>(k_max / kBlockWeights) * kXPitch + kChainWaves + 4 + kMaxChainSteps * kStepDwords) * 4;
}

uint32_t gemv_chain_max_k() { return kChainUnits * 8 * kChainThreads; }

// Fills the work split of a step for a grid of `workgroups`; false if the step does not fit the
// register slots of the resident grid.
bool gemv_chain_plan_step(ChainStep& st, uint32_t workgroups) {
    const uint32_t nb = st.k / kBlockWeights;
    st.slabs = (nb + 63) / 64;
    st.group_rows = st.epilogue == ChainStep::kSiluMulPairs ? 2 : 1;
    st.groups = st.n / st.group_rows;
    const uint32_t waves = workgroups * kChainWaves;
    const uint64_t groups_per_wave = (static_cast<uint64_t>(st.groups) + waves - 1) / waves;
    return groups_per_wave * st.group_rows * st.slabs <= static_cast<uint64_t>(kChainSlots);
}

hipError_t launch_gemv_chain(ChainArgs& args, uint32_t workgroups, uint32_t k_max, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_chain_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    args.xs_dwords = (k_max / kBlockWeights) * kXPitch;
    // more than half a CU's LDS: one workgroup per CU, so the grid spreads over all of them
    size_t lds = gemv_chain_lds_bytes(k_max);
    if (lds < 96 * 1024) lds = 96 * 1024;
    hipLaunchKernelGGL(gemv_chain_kernel, dim3(workgroups), dim3(kChainThreads), lds, stream, args);
    return hipGetLastError();
}

}  // namespace lq4
