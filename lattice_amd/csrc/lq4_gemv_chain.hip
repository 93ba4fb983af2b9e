// A chain of batch-1 GEMVs in ONE launch: the device twin of the reference encoding a whole token
// into one command buffer (forward/metal_qwen35.rs:6943 forward_step, commit at :6447; encode_mlp_block
// in inner/layers/mod.rs; the elementwise dispatches at inner/dispatch.rs:916-930, 1171-1290).  Step j is
// r_j = epilogue(W_j . prologue(x_j)); x_j is an external vector or an earlier step's result:
//   o -> (+ residual, RMSNorm) -> gate||up -> silu * up -> down -> (+ residual, RMSNorm) -> qkv ...
//
// Why one launch, and what it costs.  A 3-16 MB GEMV is over in 2-3 us, of which launch ramp, the
// first HBM round trip and the drain are most; four launches pay that four times and the memory pipe
// runs dry between them.  Here the grid is resident for the whole chain (one workgroup of eight waves
// per CU) and every wave requests the first weights of steps j+1 and j+2 before step j's result
// exists: weights do not depend on activations, only the order of the arithmetic does.  The price is
// the hand-over between steps through memory: measured on an otherwise idle chip a stored word is
// seen from another XCD after 0.55-0.8 us, but behind the weight requests that keep HBM busy, which is
// the point of the launch, the same store-then-poll takes 2.3-4.6 us.  For the decode layer of a 2B
// model (4 steps, 30 MB) this launch therefore takes 36 us where four separate launches take 16 us;
// chains of independent steps take 17.6 us.  The library runs chains step by step unless told
// otherwise (lq4_set_chain_mode); this launch is kept as the measured alternative.
//
// Work layout.  As in the batch-1 kernel a lane owns whole 20-byte blocks: lane l of a wave reads
// block 64*s + l of a row (slab s), so a wave's load pair covers 1280 contiguous bytes.  A wave works
// in units of three blocks per lane, of a shape fixed per step: three rows (K <= 2048), the gate and
// the up row of one pair (a step that ends in silu(gate) * up, K <= 2048), or three slabs of one row
// (longer rows; gate and up rows then alternate).  Rows go to waves round-robin: wave w of W takes
// rows (or pairs) w, w + W, ...  A step's first unit sits in one of two register sets that alternate
// by step, so two steps' first units can be on their way while a third step computes; further units
// of a long step ping-pong with a third set.  Every unit is six loads, whatever its shape (slots
// without work repeat a neighbour's address), so the compiler's wait counts are exact and a later
// step's loads stay in flight while an earlier step's registers are used.
//
// Hand-over.  A step's result vector goes to library scratch as 64-bit words {f32 value, launch
// epoch}, one agent-scope (coherent across the XCDs' L2s) relaxed atomic store per row; value and tag
// travel together, so a reader needs no fence and no separate flag: every workgroup polls the
// vector with agent-scope atomic loads, a wave's load covering 512 contiguous bytes, until each word
// carries this launch's epoch, then applies the prologue and stages the activations in LDS.  Polling
// waves lower their priority (s_setprio): a CU's pollers were seen to keep its memory pipe busy
// enough to hold back, for as long as they polled, the very waves whose rows they waited for.
// The epoch is a word in the context: every workgroup reads it when it starts, workgroup 0 advances
// it when it has finished, which is after every workgroup has read it as soon as the chain has one
// dependent step.  Nothing is reset between launches, so a captured launch can be replayed.  The
// wait is bounded (spin_limit polls): a wave that runs out raises the context's failure word and its
// workgroup leaves; the others run out the same way, so every kernel exits and lq4_sync reports it.
#include "lq4_b1_dev.hpp"

#include <type_traits>

namespace lq4 {

namespace {

using namespace b1;

constexpr int kChainWaves = 8;
constexpr int kChainThreads = kChainWaves * 64;
constexpr int kChainUnits = 2;  // 8-activation units per thread and step
constexpr int kUnit = 3;        // blocks per lane in a unit

constexpr uint32_t kStepDwords = sizeof(ChainStep) / 4;
static_assert(sizeof(ChainStep) == 128, "the descriptor copy assumes 32 dwords a step");

__device__ __forceinline__ unsigned long long tag_word(float v, uint32_t epoch) {
    return (static_cast<unsigned long long>(epoch) << 32) | __builtin_bit_cast(uint32_t, v);
}

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

// Unit shapes (ChainStep::shape).
constexpr int kRows3 = 0;   // slots = rows w + (3u + i) W, slab 0
constexpr int kPair = 1;    // slots = gate row, up row of pair w + u W (third slot idle), slab 0
constexpr int kSlabs3 = 2;  // slots = slabs 3 sg .. 3 sg + 2 of one row; u = entry * slab_groups + sg; entries are rows
                            // w + e W, or with pairs gate and up row of pair w + (e / 2) W in turn

// The wave-uniform facts of a step that the unit loops need.
struct StepView {
    const LQ4_GLOBAL uint8_t* w;
    uint32_t nb, row_bytes, half, n, slab_groups, pairs;
    uint32_t units;  // units of this wave in the step
};

__device__ __forceinline__ StepView view_of(const ChainStep& st, uint32_t wid, uint32_t n_waves) {
    StepView v;
    v.w = as_global(st.w);
    v.nb = st.k / kBlockWeights;
    v.row_bytes = v.nb * kBlockBytes;
    v.half = st.n / 2;
    v.n = st.n;
    v.slab_groups = (st.slabs + kUnit - 1) / kUnit;
    v.pairs = ((st.flags >> 8) & 0xff) == ChainStep::kSiluMulPairs;
    const uint32_t shape = st.flags >> 16;
    const uint32_t items = v.pairs ? v.half : st.n;  // rows or pairs dealt round-robin
    const uint32_t mine = wid < items ? (items - wid + n_waves - 1) / n_waves : 0;
    v.units = shape == kRows3 ? (mine + kUnit - 1) / kUnit : shape == kPair ? mine : mine * (v.pairs ? 2 : 1) * v.slab_groups;
    return v;
}

// Row and slab of slot i of unit u (u below the wave's unit count, except that slots of the last unit of
// a kRows3 step may lie past the last row: `row` is then clamped and `valid` false).
template <int SHAPE>
__device__ __forceinline__ void slot_of(const StepView& sv, uint32_t u, int i, uint32_t wid, uint32_t n_waves, uint32_t& row,
                                        uint32_t& slab, bool& valid) {
    if (SHAPE == kRows3) {
        row = wid + (u * kUnit + i) * n_waves;
        slab = 0;
        valid = row < sv.n;
        if (!valid) row = wid;  // the wave's first row: it has one, or no unit at all
    } else if (SHAPE == kPair) {
        row = wid + u * n_waves + (i == 1 ? sv.half : 0);
        slab = 0;
        valid = i < 2;
    } else {
        const uint32_t e = u / sv.slab_groups, sg = u - e * sv.slab_groups;
        row = sv.pairs ? wid + (e >> 1) * n_waves + ((e & 1) ? sv.half : 0) : wid + e * n_waves;
        slab = sg * kUnit + i;
        valid = slab * 64 < sv.nb;
    }
}

struct Unit {
    Q4BlockRaw b[kUnit];
};

// Six loads, always.
template <int SHAPE>
__device__ __forceinline__ void load_unit(Unit& un, const StepView& sv, uint32_t u, uint32_t wid, uint32_t n_waves, int lane) {
#pragma unroll
    for (int i = 0; i < kUnit; ++i) {
        uint32_t row, slab;
        bool valid;
        slot_of<SHAPE>(sv, u, i, wid, n_waves, row, slab, valid);
        uint32_t blk = slab * 64 + lane;
        if (blk >= sv.nb) blk = sv.nb - 1;
        const LQ4_GLOBAL uint8_t* p = sv.w + static_cast<size_t>(row) * sv.row_bytes + blk * static_cast<uint32_t>(kBlockBytes);
        un.b[i].sb = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL uint32_t*>(p));
        const u32x4u q = __builtin_nontemporal_load(reinterpret_cast<const LQ4_GLOBAL u32x4u*>(p + 4));
        un.b[i].q[0] = q.x; un.b[i].q[1] = q.y; un.b[i].q[2] = q.z; un.b[i].q[3] = q.w;
    }
}

// The same six loads for a wave without a unit in the step (or past the chain's end).  Plain cached
// loads of a line that only a few waves share: thousands of waves asking memory for ONE line with
// loads that bypass the caches were measured to stall each other for milliseconds.
__device__ __forceinline__ void load_idle(Unit& un, const LQ4_GLOBAL uint8_t* idle) {
#pragma unroll
    for (int i = 0; i < kUnit; ++i) {
        un.b[i].sb = *reinterpret_cast<const LQ4_GLOBAL uint32_t*>(idle);
        const u32x4u q = *reinterpret_cast<const LQ4_GLOBAL u32x4u*>(idle + 4);
        un.b[i].q[0] = q.x; un.b[i].q[1] = q.y; un.b[i].q[2] = q.z; un.b[i].q[3] = q.w;
    }
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
    const uint32_t n_steps = a.n_steps;
    const uint32_t n_waves = gridDim.x * kChainWaves;
    const uint32_t wid = __builtin_amdgcn_readfirstlane(blockIdx.x * kChainWaves + (tid >> 6));
    if (tid == 0) *abort_flag = 0;
    // The step descriptors are kernel arguments.  Read with scalar loads where they are needed, the
    // first touch of each of their cache lines would sit on the critical path of its step.  One
    // vector load per thread copies all of them to LDS now; the steps read them from there (same
    // address in every lane) and make them scalar again.
    {
        const uint32_t* ka = reinterpret_cast<const uint32_t*>(&a.s[0]);
        if (static_cast<uint32_t>(tid) < n_steps * kStepDwords) desc[tid] = ka[tid];
        static_assert(kMaxChainSteps * kStepDwords <= kChainThreads, "one descriptor dword per thread");
    }
    const uint32_t epoch = *as_global(a.epoch);
    const LQ4_GLOBAL uint8_t* const idle = as_global(a.idle) + (wid & 127u) * 128u;  // a.idle: 16 KB
    __builtin_amdgcn_s_setprio(3);
    __syncthreads();

    auto unit_at = [](uint32_t u) { return (u >> 2) * kBlockWeights + (u & 3) * 8; };
    auto give_up = [&](uint32_t j) {
        if (lane == 0) {
            *abort_flag = 1;
            __hip_atomic_store(as_global(a.fail), j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };

    // ---- the activations of step j: fetch (external loads, or polling earlier results) ----
    // v: the vector before the prologue's arithmetic (x, base + delta, or gate); aux: gamma or up.
    auto fetch_x = [&](const ChainStep& st, uint32_t j, float (&v)[kChainUnits][8], float (&aux)[kChainUnits][8], lds_u32* xs) {
        const uint32_t n_units = st.k / 8;
        const int prologue = st.flags & 0xff;
        // gamma / up first: they depend on nothing
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
                const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
                if (prologue == ChainStep::kAddNorm) ld8(st.gamma + unit_at(u), aux[i]);
                else if (prologue == ChainStep::kSiluMul) ld8(st.x + st.k + unit_at(u), aux[i]);
            }
        }
        // plain sources
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
                const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = 0.0f;
                if (st.base) ld8(st.base + unit_at(u), v[i]);
                if (st.x) {
                    float d[8];
                    ld8(st.x + unit_at(u), d);
                    if (st.base) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[i][e] += d[e];
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[i][e] = d[e];
                    }
                }
            }
        }
        if (!st.x_tagged && !st.base_tagged) return;
        // earlier results of this launch: poll this wave's slice until every word carries the epoch
        if (a.spin_limit == 0) {  // hand-over switched off: leave as a wave whose wait ran out does
            give_up(j);
            return;
        }
        // Word r of a lane is element (slice start) + 64 r + lane: a load instruction of the wave covers
        // 512 contiguous bytes.  (Eight consecutive words per lane would touch 64 lines per
        // instruction, and a CU's pollers would then keep its memory pipe busy enough to hold back
        // the waves that still compute the very rows being waited for.)
        float t[kChainUnits][8];
        uint32_t spins = 0;
        __builtin_amdgcn_s_setprio(0);
        while (true) {
            bool ok = true;
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i) {
                if (static_cast<uint32_t>(i * T) < n_units) {
                    const uint32_t first = (i * T + (tid & ~63)) * 8 + lane;
#pragma unroll
                    for (int r = 0; r < 8; ++r) {
                        const bool act = first + r * 64 < st.k;
                        const size_t at = act ? first + r * 64 : 0;
                        float sum = 0.0f;
                        if (st.base_tagged) {
                            const unsigned long long w = __hip_atomic_load(as_global(st.base_tagged) + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            sum = __builtin_bit_cast(float, static_cast<uint32_t>(w));
                            ok = ok && (!act || static_cast<uint32_t>(w >> 32) == epoch);
                        }
                        if (st.x_tagged) {
                            const unsigned long long w = __hip_atomic_load(as_global(st.x_tagged) + at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            const float xv_ = __builtin_bit_cast(float, static_cast<uint32_t>(w));
                            sum = st.base_tagged ? sum + xv_ : xv_;  // base + delta, in that order
                            ok = ok && (!act || static_cast<uint32_t>(w >> 32) == epoch);
                        }
                        t[i][r] = sum;
                    }
                }
            }
            if (__all(ok)) break;
            if (++spins >= a.spin_limit) {
                give_up(j);
                break;
            }
            __builtin_amdgcn_s_sleep(16);
        }
        __builtin_amdgcn_s_setprio(3);
        // Back to eight consecutive elements per lane, through the part of the destination buffer
        // that this wave is about to fill anyway (16 blocks of 36 dwords for its 512 elements), so no
        // other wave is involved and the wave's own LDS operations stay in order.
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
                const uint32_t first = (i * T + (tid & ~63)) * 8;  // the slice's first element
                LQ4_LDS float* const area = reinterpret_cast<LQ4_LDS float*>(xs + (first < st.k ? first / kBlockWeights : 0) * kXPitch);
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if (first + r * 64 + lane < st.k) area[r * 64 + lane] = t[i][r];
                typedef float f32x4 __attribute__((ext_vector_type(4)));
                const uint32_t mine = first + lane * 8 < st.k ? lane * 8 : 0;
                const f32x4 lo = *reinterpret_cast<const LQ4_LDS f32x4*>(area + mine);
                const f32x4 hi = *reinterpret_cast<const LQ4_LDS f32x4*>(area + mine + 4);
                t[i][0] = lo.x; t[i][1] = lo.y; t[i][2] = lo.z; t[i][3] = lo.w;
                t[i][4] = hi.x; t[i][5] = hi.y; t[i][6] = hi.z; t[i][7] = hi.w;
            }
        }
        // a plain base with a tagged delta: base + delta; nothing plain: the tagged sum itself
        const bool plain_part = st.base || st.x;
#pragma unroll
        for (int i = 0; i < kChainUnits; ++i) {
            if (static_cast<uint32_t>(i * T) < n_units) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = plain_part ? v[i][e] + t[i][e] : t[i][e];
            }
        }
    };

    // ---- prologue arithmetic, conversion and the LDS store; ends with the step's barrier ----
    auto finish_x = [&](const ChainStep& st, float (&v)[kChainUnits][8], const float (&aux)[kChainUnits][8], lds_u32* xs) {
        const uint32_t n_units = st.k / 8;
        const int prologue = st.flags & 0xff;
        if (prologue == ChainStep::kAddNorm) {
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i) {
                if (static_cast<uint32_t>(i * T) < n_units && tid + i * T < n_units) {
                    ss += ((v[i][0] * v[i][0] + v[i][1] * v[i][1]) + (v[i][2] * v[i][2] + v[i][3] * v[i][3])) +
                          ((v[i][4] * v[i][4] + v[i][5] * v[i][5]) + (v[i][6] * v[i][6] + v[i][7] * v[i][7]));
                    if (blockIdx.x == 0) {  // the new residual stream: for the caller, and for later steps
                        const uint32_t at = unit_at(tid + i * T);
                        if (st.resid_out) {
                            typedef float f32x4 __attribute__((ext_vector_type(4)));
                            LQ4_GLOBAL f32x4* rp = reinterpret_cast<LQ4_GLOBAL f32x4*>(as_global(st.resid_out) + at);
                            rp[0] = f32x4{v[i][0], v[i][1], v[i][2], v[i][3]};
                            rp[1] = f32x4{v[i][4], v[i][5], v[i][6], v[i][7]};
                        }
                        if (st.resid_out_tagged) {
#pragma unroll
                            for (int e = 0; e < 8; ++e)
                                __hip_atomic_store(as_global(st.resid_out_tagged) + at + e, tag_word(v[i][e], epoch),
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                    }
                }
            }
            ss = wave_sum(ss);
            if (lane == 0) red[tid >> 6] = ss;
            barrier_lds();
            float total = 0.0f;
#pragma unroll
            for (int i = 0; i < kChainWaves; i += 4) total += (red[i] + red[i + 1]) + (red[i + 2] + red[i + 3]);
            static_assert(kChainWaves % 4 == 0, "the sum of squares is combined four waves at a time");
            const float inv_rms = 1.0f / sqrtf(total / static_cast<float>(st.k) + st.eps);
#pragma unroll
            for (int i = 0; i < kChainUnits; ++i)
#pragma unroll
                for (int e = 0; e < 8; ++e) v[i][e] = v[i][e] * inv_rms * (1.0f + aux[i][e]);
        } else if (prologue == ChainStep::kSiluMul) {
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

    // ---- the first unit of step j into `un` (six loads, whatever the step's shape) ----
    auto load_first = [&](Unit& un, uint32_t j) {
        if (j < n_steps) {
            const ChainStep st = read_step(desc, j);
            const StepView sv = view_of(st, wid, n_waves);
            if (sv.units) {
                switch (st.flags >> 16) {
                    case kRows3: load_unit<kRows3>(un, sv, 0, wid, n_waves, lane); break;
                    case kPair: load_unit<kPair>(un, sv, 0, wid, n_waves, lane); break;
                    default: load_unit<kSlabs3>(un, sv, 0, wid, n_waves, lane); break;
                }
                return;
            }
        }
        load_idle(un, idle);
    };

    // ---- the arithmetic of one unit and what follows a completed row ----
    XBlock xb;
    float acc = 0.0f, v_gate = 0.0f;
    auto finish_row = [&](const ChainStep& st, const StepView& sv, float partial, uint32_t row) {
        float v = segment_sum<64>(partial);
        const int epilogue = (st.flags >> 8) & 0xff;
        uint32_t row_out = row;
        if (epilogue == ChainStep::kSiluMulPairs) {
            if (row < sv.half) {  // a gate row: kept until its up row is done
                v_gate = v;
                return;
            }
            v = silu_mul_fast(v_gate, v);
            row_out = row - sv.half;
        }
        if (lane == 63) {
            if (epilogue == ChainStep::kAddResidual) v += as_global(st.res_plain)[row];
            if (st.out_tagged)
                __hip_atomic_store(as_global(st.out_tagged) + row_out, tag_word(v, epoch), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (st.y) as_global(st.y)[row_out] = v;
            if (st.res_out) as_global(st.res_out)[row_out] = v;
        }
    };
    auto process = [&](auto shape, const Unit& un, const ChainStep& st, const StepView& sv, uint32_t u, const lds_u32* xs) {
        constexpr int SHAPE = decltype(shape)::value;
#pragma unroll
        for (int i = 0; i < kUnit; ++i) {
            uint32_t row, slab;
            bool valid;
            slot_of<SHAPE>(sv, u, i, wid, n_waves, row, slab, valid);
            if (SHAPE == kPair && i == 2) break;
            if (valid) {  // uniform across the wave
                const uint32_t blk_raw = slab * 64 + lane;
                const bool live = blk_raw < sv.nb;
                if (SHAPE == kSlabs3) load_xblock(xs, live ? blk_raw : sv.nb - 1, xb);
                acc = block_fma(un.b[i], xb, live, acc);
                if (SHAPE != kSlabs3 || (slab + 1) * 64 >= sv.nb) {  // row complete
                    finish_row(st, sv, acc, row);
                    acc = 0.0f;
                }
            }
        }
    };

    // ---- a step's units: the first one is in `first`, the others ping-pong between `other` and `first` ----
    auto run_step = [&](auto shape, Unit& first, Unit& other, const ChainStep& st, const StepView& sv, const lds_u32* xs) {
        constexpr int SHAPE = decltype(shape)::value;
        if (SHAPE != kSlabs3) load_xblock(xs, static_cast<uint32_t>(lane) < sv.nb ? lane : sv.nb - 1, xb);
        // units that have a successor request it unconditionally; the last one or two are peeled off
        uint32_t u = 0;
        for (; u + 2 < sv.units; u += 2) {
            load_unit<SHAPE>(other, sv, u + 1, wid, n_waves, lane);
            process(shape, first, st, sv, u, xs);
            load_unit<SHAPE>(first, sv, u + 2, wid, n_waves, lane);
            process(shape, other, st, sv, u + 1, xs);
        }
        if (u + 2 == sv.units) {
            load_unit<SHAPE>(other, sv, u + 1, wid, n_waves, lane);
            process(shape, first, st, sv, u, xs);
            process(shape, other, st, sv, u + 1, xs);
        } else if (u < sv.units) {
            process(shape, first, st, sv, u, xs);
        }
    };
    auto run_step_any = [&](Unit& first, Unit& other, const ChainStep& st, const StepView& sv, const lds_u32* xs) {
        if (sv.units == 0) return;
        switch (st.flags >> 16) {
            case kRows3: run_step(std::integral_constant<int, kRows3>{}, first, other, st, sv, xs); break;
            case kPair: run_step(std::integral_constant<int, kPair>{}, first, other, st, sv, xs); break;
            default: run_step(std::integral_constant<int, kSlabs3>{}, first, other, st, sv, xs); break;
        }
    };

    Unit f0, f1, pong;
    lds_u32* const xs0 = lds;
    lds_u32* const xs1 = lds + a.xs_dwords;

    // Step j's activations into LDS; between their sighting and their conversion, the first unit of
    // step j + 1 (at the start) or j + 2 goes into the free register set: the first activations are
    // requested before any weight (loads return in order), and a poll issued behind a fresh burst
    // of weight loads would only return with the last of them.
    auto enter = [&](const ChainStep& stj, uint32_t j, lds_u32* xs, Unit& free_set, uint32_t far_step, auto at_start) {
        float xv[kChainUnits][8], xaux[kChainUnits][8];
        fetch_x(stj, j, xv, xaux, xs);
        load_first(free_set, far_step);
        if constexpr (decltype(at_start)::value) load_first(f1, 1);
        const bool ok = finish_x(stj, xv, xaux, xs);
        return ok;
    };

    ChainStep st = read_step(desc, 0);
    if (!enter(st, 0, xs0, f0, 0, std::true_type{})) return;
    for (uint32_t j = 0; j < n_steps; j += 2) {
        {
            const StepView sv = view_of(st, wid, n_waves);
            run_step_any(f0, pong, st, sv, xs0);
            }
        if (j + 1 >= n_steps) break;
        st = read_step(desc, j + 1);
        if (!enter(st, j + 1, xs1, f0, j + 2, std::false_type{})) return;
        {
            const StepView sv = view_of(st, wid, n_waves);
            run_step_any(f1, pong, st, sv, xs1);
            }
        if (j + 2 >= n_steps) break;
        st = read_step(desc, j + 2);
        if (!enter(st, j + 2, xs0, f1, j + 3, std::false_type{})) return;
    }
    // every workgroup read the epoch before workgroup 0 could get here through a dependent step
    if (blockIdx.x == 0 && tid == 0)
        __hip_atomic_store(as_global(a.epoch), epoch + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace

size_t gemv_chain_lds_bytes(uint32_t k_max) {
    // two activation buffers | sums of squares | abort word (+ padding) | step descriptors
    return (2 * static_cast<size_t>(k_max / kBlockWeights) * kXPitch + kChainWaves + 4 + kMaxChainSteps * kStepDwords) * 4;
}

uint32_t gemv_chain_max_k() { return kChainUnits * 8 * kChainThreads; }

// Fills the work split of a step: slabs and, in the top half of flags, the unit shape.
void gemv_chain_plan_step(ChainStep& st) {
    const uint32_t nb = st.k / kBlockWeights;
    const uint32_t epilogue = (st.flags >> 8) & 0xff;
    st.slabs = (nb + 63) / 64;
    const uint32_t shape = st.slabs > 1 ? kSlabs3 : epilogue == ChainStep::kSiluMulPairs ? kPair : kRows3;
    st.flags = (st.flags & 0xffff) | (shape << 16);
    st.groups = 0;
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
