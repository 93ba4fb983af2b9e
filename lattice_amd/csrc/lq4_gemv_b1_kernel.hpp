#pragma once
// Batch-1 decode GEMV, the bandwidth-critical kernel:  y[n] = sum_k W[n,k] * x[k].
//
// Work layout.  A "slab" is 64 consecutive blocks of one weight row (2048 weights,
// 1280 contiguous bytes).  Lane l of a wave owns block 64*s + l of every row the wave
// processes, so one load-instruction pair per lane (dwordx4 + dword) covers a whole slab
// with no byte fetched twice, and the 32 activations a lane needs are the same for every
// row: they are staged once per workgroup in LDS and held in registers across rows.
// Rows shorter than a slab (K = 1024 or 512) put 2 or 4 rows side by side in one wave.
// Waves are persistent: each walks a strided list of row groups and keeps the next
// group's blocks in flight while it works on the current one.
//
// The unpack-free arithmetic (eight-wide 4-bit dot products of a packed dword with the digits of per-block
// scaled fixed-point activations) and the LDS staging are in lq4_b1_dev.hpp, shared with the decode-chain
// kernel and the per-pair MoE kernels.
#include "lq4_b1_dev.hpp"

#include <type_traits>

namespace lq4 {

namespace {

using namespace b1;

constexpr int kWaves = 4;  // waves per workgroup unless a launch asks for more

// A wave-row is 64/SEG weight rows side by side (SEG lanes each).  Wave `wid` of `n_waves`
// works through chunks of RW wave-rows — chunk c holds wave-rows (c*RW + j)*n_waves + wid,
// j < RW (with several chunks per wave: (c*n_waves + wid)*RW + j) — and, inside a chunk, through
// groups of SG slabs.  One (chunk, slab group) is a
// unit: RW*SG blocks per lane, loaded with one burst; the next unit's burst is in flight
// while the current one is consumed.  Dynamic LDS: (K/32) * kXPitch dwords.
//
// FUSED instantiations take a GemvFusion: the activations are produced while they are staged
// (residual add + shifted RMSNorm, or silu(gate) * up) and the result can be added into a
// residual stream as it is stored.  Every workgroup stages the whole activation vector anyway,
// so the norm costs one extra pass over K floats per workgroup and no launch.
// Whole-wave call.  Returns t[lane] (0 beyond the rank) once every slot carries this launch's tag; polls the
// slots at most `spin_limit` times and otherwise computes t in this wave.  The slots are read with
// agent-scope atomic loads (they do not hit in this XCD's caches), value and tag in one word.
// The wave that computes t itself follows the producers' summation exactly (the k partition of a
// WAVES*64-thread workgroup, the same wave sum, then the waves' sums in order), so t has the same
// bits whichever way a wave obtained it.  Such waves count themselves in sync[2].
// `a_row(j)` names row j of A: {matrix, its dtype flag, row inside it} (one matrix, or several stacked).
struct LoraARow {
    const void* a;
    int is_f16;
    uint32_t j;
};
template <int WAVES, typename ARowOf>
__device__ __forceinline__ float lora_t_acquire(const LoraEpilogue& lora, uint32_t tag, uint32_t k,
                                                const float* __restrict__ x, int lane, ARowOf a_row) {
    const bool mine = static_cast<uint32_t>(lane) < lora.rank;
    const unsigned long long none = static_cast<unsigned long long>(tag) << 32;  // lanes beyond the rank: as if published
    if (lora.spin_limit) {
        // First look through the caches: when the producers are done, which is the usual case, the
        // line is fetched once per XCD instead of once per wave.  A line cached too early is only
        // incomplete (its tags say so) and the polls below go past the caches.
        unsigned long long v = none;
        if (mine) v = *static_cast<const volatile unsigned long long*>(&lora.slots[lane]);
        if (__all(static_cast<uint32_t>(v >> 32) == tag)) return __builtin_bit_cast(float, static_cast<uint32_t>(v));
    }
    for (uint32_t spin = 0; spin < lora.spin_limit; ++spin) {
        unsigned long long v = none;
        if (mine) v = __hip_atomic_load(&lora.slots[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__all(static_cast<uint32_t>(v >> 32) == tag)) return __builtin_bit_cast(float, static_cast<uint32_t>(v));
        __builtin_amdgcn_s_sleep(4);
    }
    if (lane == 0) __hip_atomic_fetch_add(&lora.sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float t = 0.0f;
    for (uint32_t j = 0; j < lora.rank; ++j) {
        float total = 0.0f;
        const LoraARow ar = a_row(j);
#pragma unroll
        for (int v = 0; v < WAVES; ++v)
            total += wave_sum(lora_a_row_partial(ar.a, ar.is_f16, ar.j, k, x, v * 64 + lane, WAVES * 64));
        if (static_cast<uint32_t>(lane) == j) t = total;
    }
    return t;
}

struct NoFusion {};
template <int MODE>
struct FusionArg {
    typedef NoFusion type;
};
template <>
struct FusionArg<1> {
    typedef GemvFusion type;
};
template <>
struct FusionArg<5> {
    typedef GemvFusion type;
};
template <>
struct FusionArg<6> {
    typedef MultiViews type;
};
template <>
struct FusionArg<7> {
    typedef MultiViews type;
};

// WAVES: waves per workgroup.  Every workgroup stages the whole activation vector, so on long rows
// (K of 4096..8192) eight waves share one staging where four would each pay half of it again.
//
// MODE: 0 plain, 1 fused prologue/epilogue (GemvFusion), 2 plain with the LoRA factor t = A.x
// computed inside the launch: workgroups 0..rank-1 each reduce one row of A against x and publish
// it under the launch's tag, the weight workgroups behind them pick t up when their first rows are
// complete, as a rule long after it was published.  The wait is bounded: a wave that runs out of polls
// computes t itself, so every wave finishes whatever the dispatch order was.
// 4 plain, with the row order of a persistent grid (see ADJ below).
// 6 several matrices with rows of the same K against one x (MultiViews): the launch walks the rows of the matrices
// stacked one under the other, view v holding rows [begin[v], begin[v + 1]); a wave-row never straddles two views
// (the launcher sees to it), so the view of a wave-row is uniform across the wave.  Each view has its own output
// and its own LoRA epilogue (t = A . x from memory).
// 7 the same with the adapters' factors computed inside the launch as in mode 2: the A matrices of the views
// stacked (at most 64 rows in all), one producer workgroup a row in front of the weight workgroups; lane l of a
// weight wave picks up t of stacked row l, view v's factors start at lane t_off[v].
constexpr int kPlainMode = 0, kFusedMode = 1, kLoraAMode = 2, kPlainAdjMode = 4, kFusedPairsMode = 5,
              kMultiMode = 6, kMultiLoraAMode = 7;

template <int RW, int SG, int SEG, int MODE, int WAVES = kWaves>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4_b1(const uint8_t* __restrict__ w, uint32_t n,
                                                          uint32_t k, const float* __restrict__ x,
                                                          float* __restrict__ y, LoraEpilogue lora,
                                                          typename FusionArg<MODE>::type fz) {
    extern __shared__ __attribute__((aligned(16))) uint32_t xs[];
    lds_u32* const xsl = (lds_u32*)xs;
    constexpr bool FUSED = MODE == kFusedMode || MODE == kFusedPairsMode;
    constexpr bool PAIRS = MODE == kFusedPairsMode;  // fused, with the kSiluMulPairs epilogue (a mode of its own:
                                                     // as a run-time flag it doubled the time of every fused launch)
    constexpr bool MINA = MODE == kMultiLoraAMode;            // several views, A . x inside the launch
    constexpr bool INA = MODE == kLoraAMode || MINA;          // producer workgroups in front
    constexpr bool MULTI = MODE == kMultiMode || MINA;
    constexpr int RPW = 64 / SEG;  // weight rows per wave-row
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // workgroups that stream weights, and this one's index among them
    uint32_t w_groups = gridDim.x, w_group = blockIdx.x;
    // where row j of the (stacked) A lives
    auto a_row = [&](uint32_t j) {
        if constexpr (MINA) {
            uint32_t v = 0;
#pragma unroll
            for (int i = 1; i < kMaxViews; ++i) v += (static_cast<uint32_t>(i) < fz.count && j >= fz.t_off[i]) ? 1u : 0u;
            return LoraARow{fz.a[v], fz.b_is_f16[v], j - fz.t_off[v]};
        } else {
            return LoraARow{lora.a, lora.b_is_f16, j};
        }
    };
    if constexpr (INA) {
        if (blockIdx.x < lora.rank) {  // ---- one row of A against x ----
            const LoraARow ar = a_row(blockIdx.x);
            const float p = lora_a_row_partial(ar.a, ar.is_f16, ar.j, k, x, tid, WAVES * 64);
            const float ws = wave_sum(p);
            float* part = reinterpret_cast<float*>(xs);
            if (lane == 0) part[tid >> 6] = ws;
            __syncthreads();
            if (tid == 0) {
                float total = 0.0f;
#pragma unroll
                for (int i = 0; i < WAVES; ++i) total += part[i];
                const unsigned long long word = (static_cast<unsigned long long>(launch_tag()) << 32) | __builtin_bit_cast(uint32_t, total);
                __hip_atomic_store(&lora.slots[blockIdx.x], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            return;
        }
        w_groups -= lora.rank;
        w_group -= lora.rank;
    }
    const int sub = lane / SEG;   // which of the side-by-side rows
    const int seg_lane = lane % SEG;
    const uint32_t nb = k / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t slabs = SEG == 64 ? (nb + 63) / 64 : 1;
    const uint32_t slab_groups = (slabs + SG - 1) / SG;
    const uint32_t n_wrows = (n + RPW - 1) / RPW;
    const uint32_t n_waves = w_groups * WAVES;
    // the wave index is uniform across the wave: keep it (and everything derived) scalar
    const uint32_t wid = __builtin_amdgcn_readfirstlane(w_group * WAVES + (tid >> 6));
    // chunks whose first wave-row exists for this wave (later waves may have one chunk fewer)
    const uint32_t first = wid < n_wrows ? n_wrows - wid : 0;  // wave-rows from this wave's first one on
    uint32_t chunks = (first + n_waves * RW - 1) / (n_waves * RW);
    // kPlainAdjMode, for a persistent grid (waves that walk several chunks): the RW wave-rows of a chunk lie next
    // to each other in memory, chunk c of wave wid = wave-rows (c * n_waves + wid) * RW + j, so the wave's requests
    // of one unit fall into one run of RW rows (lm_head 63.4 -> 60.6 us in the same run on one device).  With one
    // chunk per wave the interleaved order is the faster one (12288 x 2048 5.25 against 5.46 us, 2048 x 6144 3.8
    // against 4.1), and the choice as a run-time flag cost those launches 6-11 %: hence a mode of its own.
    constexpr bool ADJ = MODE == kPlainAdjMode;
    if constexpr (ADJ) chunks = wid * RW < n_wrows ? (n_wrows - wid * RW + n_waves * RW - 1) / (n_waves * RW) : 0;
    // Fused epilogue kSiluMulPairs (W = [gate rows | up rows], n / 2 of each; rows of 64 lanes, RW even): the
    // wave's rounds come in pairs, rounds 2i and 2i + 1 are the gate and the up row of pair i * n_waves + wid, so
    // that the wave itself forms silu(g) * u when the second row of a pair completes.
    static_assert(!PAIRS || (RW % 2 == 0 && SEG == 64), "pairs: chunks of whole pairs, rows of 64 lanes");
    const uint32_t n_pairs = n / 2;
    if constexpr (PAIRS) {
        const uint32_t mine = wid < n_pairs ? (n_pairs - wid + n_waves - 1) / n_waves : 0;
        chunks = (2 * mine + RW - 1) / RW;
    }
    // wave-row of round r = chunk * RW + j, and whether this wave owns it
    auto wrow_of = [&](uint32_t r) {
        if (PAIRS) {
            const uint32_t pair = (r >> 1) * n_waves + wid;
            return (r & 1) ? n_pairs + pair : pair;  // (a pair past the end: past n, or an up row; clamped or dropped)
        }
        return ADJ ? (r / RW) * (n_waves * RW) + wid * RW + r % RW : r * n_waves + wid;
    };
    auto wrow_mine = [&](uint32_t r) {
        if (PAIRS) return (r >> 1) * n_waves + wid < n_pairs;
        return wrow_of(r) < n_wrows;
    };
    const uint32_t units = chunks * slab_groups;
    // kMultiMode: the view that holds stacked row `row` (uniform: called with the first row of a wave-row)
    auto view_of = [&](uint32_t row) {
        uint32_t v = 0;
        if constexpr (MULTI) {
#pragma unroll
            for (int i = 1; i < kMaxViews; ++i) v += (static_cast<uint32_t>(i) < fz.count && row >= fz.begin[i]) ? 1u : 0u;
        }
        return v;
    };

    // ---- the first activations are requested before any weight so they can be waited on alone ----
    // (straight-line code, clamped addresses: no branch between the loads and their wait).  Loads
    // return in order: an activation load issued after the weight prefetch would hold its staging,
    // and the barrier behind it, back until the first weights have crossed from HBM.  Rows longer
    // than one slab hoist more 8-activation units per thread: two with eight waves (all of K up to
    // 8192), eight with four waves (rows beyond that; measured, 5120 x 17408 18.0 -> 16.4 us).
    constexpr int HX = SG < 2 ? 1 : WAVES == 8 ? 2 : 8;
    // fused prologues hold up to four vectors per unit, so they hoist at most three units
    constexpr int HF = FUSED ? (HX < 3 ? HX : 3) : HX;
    uint32_t gx[HF];
    float4 xa[HF], xb[HF];  // plain: x;  add + norm: base (+ delta);  silu * up: gate
    float4 ya[FUSED ? HF : 1], yb[FUSED ? HF : 1];  // add + norm: gamma;  silu * up: up
#pragma unroll
    for (int i = 0; i < HF; ++i) {
        const uint32_t g = tid + i * WAVES * 64;
        gx[i] = g < nb * 4 ? g : 0;
        const uint32_t at = (gx[i] >> 2) * kBlockWeights + (gx[i] & 3) * 8;
        if constexpr (!FUSED) {
            const float4* xp = reinterpret_cast<const float4*>(x + at);
            xa[i] = xp[0];
            xb[i] = xp[1];
        } else if (fz.prologue == GemvFusion::kAddNorm) {
            const float4* bp = reinterpret_cast<const float4*>(fz.base + at);
            xa[i] = bp[0];
            xb[i] = bp[1];
            if (fz.delta) {
                const float4* dp = reinterpret_cast<const float4*>(fz.delta + at);
                const float4 da = dp[0], db = dp[1];
                xa[i].x += da.x; xa[i].y += da.y; xa[i].z += da.z; xa[i].w += da.w;
                xb[i].x += db.x; xb[i].y += db.y; xb[i].z += db.z; xb[i].w += db.w;
            }
            const float4* gp = reinterpret_cast<const float4*>(fz.gamma + at);
            ya[i] = gp[0];
            yb[i] = gp[1];
        } else if (fz.prologue == GemvFusion::kSiluMul) {
            const float4* gp = reinterpret_cast<const float4*>(x + at);
            const float4* up = reinterpret_cast<const float4*>(x + k + at);
            xa[i] = gp[0];
            xb[i] = gp[1];
            ya[i] = up[0];
            yb[i] = up[1];
        } else {
            const float4* xp = reinterpret_cast<const float4*>(x + at);
            xa[i] = xp[0];
            xb[i] = xp[1];
            ya[i] = xa[i];
            yb[i] = xb[i];
        }
    }

    // Loads unit u's blocks.  Lanes past the end of a row and rows past N re-read a valid
    // block; their contribution is zeroed or dropped later.
    auto load_unit = [&](Q4BlockRaw (&buf)[RW][SG], uint32_t u) {
        const uint32_t chunk = u / slab_groups, sgi = u - chunk * slab_groups;
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            uint32_t wrow = wrow_of(chunk * RW + j);  // scalar
            if (wrow >= n_wrows) wrow = n_wrows - 1;
            uint32_t row = wrow * RPW + sub;
            if (RPW > 1 && row >= n) row = n - 1;
            const uint8_t* rp = w + row * row_bytes;  // scalar base when RPW == 1
            if constexpr (MULTI) {
                const uint32_t v = view_of(wrow * RPW);
                rp = fz.w[v] + (row - fz.begin[v]) * row_bytes;
            }
#pragma unroll
            for (int t = 0; t < SG; ++t) {
                uint32_t blk = (sgi * SG + t) * 64 + seg_lane;
                if (blk >= nb) blk = nb - 1;
                // non-temporal: every block is read once, and a plain load's allocation in the caches
                // measurably slows the stream (read probe: 4.9 -> 5.15 TB/s at 30 MB, 6.2 -> 6.8 at 318 MB)
                const uint8_t* bp = rp + blk * static_cast<uint32_t>(kBlockBytes);
                buf[j][t].sb = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(bp));
                const u32x4u q = __builtin_nontemporal_load(reinterpret_cast<const u32x4u*>(bp + 4));
                buf[j][t].q[0] = q.x; buf[j][t].q[1] = q.y; buf[j][t].q[2] = q.z; buf[j][t].q[3] = q.w;
            }
        }
    };

    // LoRA factors of the first chunk's rows (lane i of a row holds t[i] and B[row, i]), requested ahead
    // of the weights like the activations: fetched only when the chunk completes, they would add a
    // memory round trip to the tail of the kernel
    float lora_t0 = 0.0f, lora_b0[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) lora_b0[j] = 0.0f;
    if (!MULTI && lora.rank && static_cast<uint32_t>(seg_lane) < lora.rank) {
        if constexpr (!INA) lora_t0 = lora.t[seg_lane];
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const uint32_t wrow = wrow_of(j);
            uint32_t row = wrow * RPW + sub;
            row = (wrow < n_wrows && row < n) ? row : n - 1;
            const size_t bi = static_cast<size_t>(row) * lora.rank + seg_lane;
            lora_b0[j] = lora.b_is_f16 ? static_cast<float>(static_cast<const _Float16*>(lora.b)[bi])
                                       : static_cast<const float*>(lora.b)[bi];
        }
    }

    // kMultiMode: the same for each row's own view
    float multi_t0[MULTI ? RW : 1], multi_b0[MULTI ? RW : 1];
    if constexpr (MULTI) {
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            multi_t0[j] = 0.0f;
            multi_b0[j] = 0.0f;
            uint32_t wrow = wrow_of(j);
            if (wrow >= n_wrows) wrow = n_wrows - 1;
            uint32_t row = wrow * RPW + sub;
            if (RPW > 1 && row >= n) row = n - 1;
            const uint32_t v = view_of(wrow * RPW);
            const uint32_t rank = fz.rank[v];
            if (static_cast<uint32_t>(seg_lane) < rank) {
                const size_t bi = static_cast<size_t>(row - fz.begin[v]) * rank + seg_lane;
                multi_b0[j] = fz.b_is_f16[v] ? static_cast<float>(static_cast<const _Float16*>(fz.b[v])[bi])
                                             : static_cast<const float*>(fz.b[v])[bi];
                if constexpr (!MINA) multi_t0[j] = fz.t[v][seg_lane];
            }
        }
    }

    Q4BlockRaw buf_a[RW][SG], buf_b[RW][SG];
    load_unit(buf_a, 0);
    // residual values of the first chunk's rows, requested now so the final store does not wait
    float res_first[RW];
    if constexpr (FUSED) {
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const uint32_t wrow = wrow_of(j);
            const uint32_t row = wrow * RPW + sub;
            res_first[j] = (fz.epilogue == GemvFusion::kAddResidual && wrow < n_wrows && row < n) ? fz.residual[row] : 0.0f;
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads

    // ---- stage x: thread handles (block, dword j) = 8 activations ---------------------------
    auto stage = [&](uint32_t g, const float4 a, const float4 b, bool store) { stage_x8(xsl, g, a, b, store); };
    if constexpr (!FUSED) {
#pragma unroll
        for (int i = 0; i < HF; ++i) stage(gx[i], xa[i], xb[i], tid + i * WAVES * 64 < nb * 4);
        for (uint32_t g = tid + HF * WAVES * 64; g < nb * 4; g += WAVES * 64) {
            const float4* xp = reinterpret_cast<const float4*>(x + (g >> 2) * kBlockWeights + (g & 3) * 8);
            stage(g, xp[0], xp[1], true);
        }
    } else {
        __shared__ float red[WAVES];
        const uint32_t n_units = nb * 4;
        auto unit_at = [](uint32_t g) { return (g >> 2) * kBlockWeights + (g & 3) * 8; };
        auto add4 = [](float4 a, const float4 b) {
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
            return a;
        };
        auto sq4 = [](const float4 a) { return (a.x * a.x + a.y * a.y) + (a.z * a.z + a.w * a.w); };
        auto norm4 = [](float4 v, float inv, const float4 g) {
            v.x = v.x * inv * (1.0f + g.x); v.y = v.y * inv * (1.0f + g.y);
            v.z = v.z * inv * (1.0f + g.z); v.w = v.w * inv * (1.0f + g.w);
            return v;
        };
        // v = base + delta for unit g (8 activations)
        auto load_v = [&](uint32_t g, float4& a, float4& b) {
            const float4* bp = reinterpret_cast<const float4*>(fz.base + unit_at(g));
            a = bp[0];
            b = bp[1];
            if (fz.delta) {
                const float4* dp = reinterpret_cast<const float4*>(fz.delta + unit_at(g));
                a = add4(a, dp[0]);
                b = add4(b, dp[1]);
            }
        };
        if (fz.prologue == GemvFusion::kAddNorm) {
            // The hoisted units of a thread stay in registers between the sum of squares and the
            // scaling, with their gamma; longer vectors re-read the rest.
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < HF; ++i) {
                const uint32_t g = tid + i * WAVES * 64;
                if (g < n_units) {
                    ss += sq4(xa[i]) + sq4(xb[i]);
                    if (blockIdx.x == 0 && fz.residual_out) {
                        float4* rp = reinterpret_cast<float4*>(fz.residual_out + unit_at(g));
                        rp[0] = xa[i];
                        rp[1] = xb[i];
                    }
                }
            }
            for (uint32_t g = tid + HF * WAVES * 64; g < n_units; g += WAVES * 64) {
                float4 a, b;
                load_v(g, a, b);
                ss += sq4(a) + sq4(b);
                if (blockIdx.x == 0 && fz.residual_out) {
                    float4* rp = reinterpret_cast<float4*>(fz.residual_out + unit_at(g));
                    rp[0] = a;
                    rp[1] = b;
                }
            }
            ss = wave_sum(ss);
            if (lane == 0) red[tid >> 6] = ss;
            __syncthreads();
            float total = (red[0] + red[1]) + (red[2] + red[3]);
            if constexpr (WAVES == 8) total += (red[4] + red[5]) + (red[6] + red[7]);
            static_assert(WAVES == 4 || WAVES == 8, "the sum of squares is combined for four or eight waves");
            const float inv_rms = 1.0f / sqrtf(total / static_cast<float>(k) + fz.eps);
#pragma unroll
            for (int i = 0; i < HF; ++i)
                stage(gx[i], norm4(xa[i], inv_rms, ya[i]), norm4(xb[i], inv_rms, yb[i]), tid + i * WAVES * 64 < n_units);
            for (uint32_t g = tid + HF * WAVES * 64; g < n_units; g += WAVES * 64) {
                float4 a, b;
                load_v(g, a, b);
                const float4* gp = reinterpret_cast<const float4*>(fz.gamma + unit_at(g));
                stage(g, norm4(a, inv_rms, gp[0]), norm4(b, inv_rms, gp[1]), true);
            }
        } else if (fz.prologue == GemvFusion::kSiluMul) {
            // silu through the hardware exp2 and reciprocal (about 1 ulp each): every workgroup
            // evaluates the whole vector, so the library expf and an IEEE divide would sit on
            // the critical path of each of them.
            auto silu_mul = [](float gate, float u) {
                const float e = __builtin_amdgcn_exp2f(gate * -1.44269504088896340736f);
                return gate * __builtin_amdgcn_rcpf(1.0f + e) * u;
            };
            auto silu_mul8 = [&](const float4 ga, const float4 gb, const float4 ua, const float4 ub, float4& a, float4& b) {
                a.x = silu_mul(ga.x, ua.x); a.y = silu_mul(ga.y, ua.y); a.z = silu_mul(ga.z, ua.z); a.w = silu_mul(ga.w, ua.w);
                b.x = silu_mul(gb.x, ub.x); b.y = silu_mul(gb.y, ub.y); b.z = silu_mul(gb.z, ub.z); b.w = silu_mul(gb.w, ub.w);
            };
#pragma unroll
            for (int i = 0; i < HF; ++i) {
                float4 a, b;
                silu_mul8(xa[i], xb[i], ya[i], yb[i], a, b);
                stage(gx[i], a, b, tid + i * WAVES * 64 < n_units);
            }
            for (uint32_t g = tid + HF * WAVES * 64; g < n_units; g += WAVES * 64) {
                const float4* gp = reinterpret_cast<const float4*>(x + unit_at(g));
                const float4* up = reinterpret_cast<const float4*>(x + k + unit_at(g));
                float4 a, b;
                silu_mul8(gp[0], gp[1], up[0], up[1], a, b);
                stage(g, a, b, true);
            }
        } else {
#pragma unroll
            for (int i = 0; i < HF; ++i) stage(gx[i], xa[i], xb[i], tid + i * WAVES * 64 < n_units);
            for (uint32_t g = tid + HF * WAVES * 64; g < n_units; g += WAVES * 64) {
                const float4* xp = reinterpret_cast<const float4*>(x + unit_at(g));
                stage(g, xp[0], xp[1], true);
            }
        }
    }
    __syncthreads();

    float acc[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) acc[j] = 0.0f;
    float gate_kept = 0.0f;                  // kSiluMulPairs: the gate row's sum until the pair's up row is done
    float t_reg = 0.0f;   // kLoraAMode: t[lane], fetched when the wave's first rows are complete
    bool t_have = false;

    // Consumes unit u from `cur` while unit u+1 streams into `nxt`.
    // `prefetch` is a compile-time flag: a load behind a run-time condition would make the compiler
    // wait, before the current unit's blocks are used, for as many loads as the path WITHOUT the
    // prefetch needs, i.e. for most of the just-issued next unit as well.
    auto process = [&](auto prefetch, Q4BlockRaw (&cur)[RW][SG], Q4BlockRaw (&nxt)[RW][SG], uint32_t u) {
        const uint32_t chunk = u / slab_groups, sgi = u - chunk * slab_groups;
        if constexpr (decltype(prefetch)::value) load_unit(nxt, u + 1);

#pragma unroll
        for (int t = 0; t < SG; ++t) {
            const uint32_t slab = sgi * SG + t;
            if (slab < slabs) {  // uniform across the wave
                const uint32_t blk_raw = slab * 64 + seg_lane;
                const bool live = blk_raw < nb;
                const uint32_t blk = live ? blk_raw : nb - 1;
                XBlock xblk;
                load_xblock(xsl, blk, xblk);
#pragma unroll
                for (int j = 0; j < RW; ++j) acc[j] = block_fma(cur[j][t], xblk, live, acc[j]);
            }
        }

        if (sgi + 1 == slab_groups) {  // chunk complete: reduce and store its rows
#pragma unroll
            for (int j = 0; j < RW; ++j) {
                const uint32_t wrow = wrow_of(chunk * RW + j);
                const uint32_t row = wrow * RPW + sub;
                const bool row_ok = wrow_mine(chunk * RW + j) && row < n;
                float v = acc[j];
                acc[j] = 0.0f;
                if constexpr (INA) {
                    // lane l of the wave holds t[l]; every lane takes part in the exchange
                    if (!t_have) {
                        t_reg = lora_t_acquire<WAVES>(lora, launch_tag(), k, x, lane, a_row);
                        t_have = true;
                    }
                    // the adapter of this row: the launch's one, or (several views) the one of the row's view, whose
                    // factors start at lane t_off of the stacked t
                    uint32_t e_rank = lora.rank, e_off = 0, e_row = row;
                    float e_scale = lora.scale;
                    const void* e_b = lora.b;
                    int e_f16 = lora.b_is_f16;
                    if constexpr (MINA) {
                        const uint32_t vw = view_of((wrow < n_wrows ? wrow : n_wrows - 1) * RPW);
                        e_rank = fz.rank[vw];
                        e_off = fz.t_off[vw];
                        e_row = row - fz.begin[vw];
                        e_scale = fz.scale[vw];
                        e_b = fz.b[vw];
                        e_f16 = fz.b_is_f16[vw];
                    }
                    for (uint32_t i0 = 0; i0 < e_rank; i0 += SEG) {
                        const uint32_t i = i0 + seg_lane;
                        const float ti = __shfl(t_reg, static_cast<int>((e_off + i) & 63u), 64);
                        if (row_ok && i < e_rank) {
                            float bv;
                            if (chunk == 0 && i0 == 0) {
                                bv = MINA ? multi_b0[j] : lora_b0[j];  // requested at kernel start
                            } else {
                                const size_t bi = static_cast<size_t>(e_row) * e_rank + i;
                                bv = e_f16 ? static_cast<float>(static_cast<const _Float16*>(e_b)[bi])
                                           : static_cast<const float*>(e_b)[bi];
                            }
                            v = fmaf(e_scale * bv, ti, v);
                        }
                    }
                } else if constexpr (MULTI) {
                    const uint32_t vw = view_of((wrow < n_wrows ? wrow : n_wrows - 1) * RPW);
                    const uint32_t rank = fz.rank[vw];
                    if (rank && row_ok) {
                        const float scale = fz.scale[vw];
                        uint32_t i = seg_lane;
                        if (chunk == 0 && i < rank) {  // requested at kernel start
                            v = fmaf(scale * multi_b0[j], multi_t0[j], v);
                            i += SEG;
                        }
                        for (; i < rank; i += SEG) {
                            const size_t bi = static_cast<size_t>(row - fz.begin[vw]) * rank + i;
                            const float bv = fz.b_is_f16[vw] ? static_cast<float>(static_cast<const _Float16*>(fz.b[vw])[bi])
                                                             : static_cast<const float*>(fz.b[vw])[bi];
                            v = fmaf(scale * bv, fz.t[vw][i], v);
                        }
                    }
                } else if (lora.rank && row_ok) {
                    // the row's lanes share out scale * B[row, i] * t[i]; the sum below folds it in
                    uint32_t i = seg_lane;
                    if (chunk == 0 && i < lora.rank) {  // requested at kernel start
                        v = fmaf(lora.scale * lora_b0[j], lora_t0, v);
                        i += SEG;
                    }
                    for (; i < lora.rank; i += SEG) {
                        const size_t bi = static_cast<size_t>(row) * lora.rank + i;
                        const float bv = lora.b_is_f16 ? static_cast<float>(static_cast<const _Float16*>(lora.b)[bi])
                                                       : static_cast<const float*>(lora.b)[bi];
                        v = fmaf(lora.scale * bv, lora.t[i], v);
                    }
                }
                v = segment_sum<SEG>(v);
                if constexpr (PAIRS) {
                    if (j % 2 == 0) {
                        gate_kept = v;
                    } else if (seg_lane == SEG - 1 && row_ok) {
                        // silu through the hardware exp2 and reciprocal, the form the staging of a
                        // [gate | up] vector uses
                        const float e = __builtin_amdgcn_exp2f(gate_kept * -1.44269504088896340736f);
                        y[row - n_pairs] = gate_kept * __builtin_amdgcn_rcpf(1.0f + e) * v;
                    }
                    continue;
                }
                if (seg_lane == SEG - 1 && row_ok) {
                    if constexpr (FUSED) {
                        if (y) y[row] = v;
                        if (fz.epilogue == GemvFusion::kAddResidual) {
                            const float r = (chunk == 0 ? res_first[j] : fz.residual[row]) + v;
                            fz.residual[row] = r;
                            if (fz.copy_dst) fz.copy_dst[row] = r;
                        }
                    } else if constexpr (MULTI) {
                        const uint32_t vw = view_of(wrow * RPW);  // (row_ok: the wave-row exists)
                        fz.y[vw][row - fz.begin[vw]] = v;
                    } else {
                        y[row] = v;
                    }
                }
            }
        }
    };

    // two buffers swap roles every unit, so no block is ever copied between registers
    // (units that have a successor prefetch it unconditionally; the last one or two are peeled off)
    constexpr std::true_type kFetch{};
    constexpr std::false_type kLast{};
    uint32_t u = 0;
    for (; u + 2 < units; u += 2) {
        process(kFetch, buf_a, buf_b, u);
        process(kFetch, buf_b, buf_a, u + 1);
    }
    if (u + 2 == units) {
        process(kFetch, buf_a, buf_b, u);
        process(kLast, buf_b, buf_a, u + 1);
    } else if (u < units) {
        process(kLast, buf_a, buf_b, u);
    }

}

// Grid shape of one launch: waves in all, wave-rows per chunk, slabs per unit.
struct B1Plan {
    size_t lds;
    uint32_t seg, wg_waves, waves, rw, sg;
    bool persistent;  // waves walk several chunks
};

// `producers`: workgroups in front of the weight workgroups.  `four_waves`: never the eight-wave
// workgroups.  `lds_min`: dynamic LDS the launch needs beyond the staged x.  `even_rw`: chunks of two or four
// wave-rows only (the kSiluMulPairs epilogue).
B1Plan plan_b1(uint32_t n, uint32_t k, uint32_t producers, bool four_waves, size_t lds_min, bool even_rw = false) {
    B1Plan p;
    p.lds = gemv_b1_lds_bytes(k);
    if (p.lds < lds_min) p.lds = lds_min;
    const size_t lds = p.lds;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t seg = nb == 32 ? 32 : nb == 16 ? 16 : 64;
    const uint32_t n_wrows = (n + 64 / seg - 1) / (64 / seg);
    const uint32_t slabs = seg == 64 ? (nb + 63) / 64 : 1;
    // Up to 16 waves per CU (4096 in all), fewer when the staged x leaves room for fewer
    // workgroups; rows per wave chosen so every wave gets the same share (to within one).
    uint32_t wg_per_cu = static_cast<uint32_t>((160 * 1024) / (lds + 512));
    // eight waves per workgroup on long rows (measured: 2048 x 6144 5.15 -> 4.69 us, 17408 x 5120
    // 16.2 -> 15.2; behind on K 2048 and K 17408)
    const uint32_t wg_waves = (!four_waves && seg == 64 && k >= 4096 && k <= 8192) ? 8 : kWaves;
    wg_per_cu = wg_per_cu > 16 / wg_waves ? 16 / wg_waves : wg_per_cu < 1 ? 1 : wg_per_cu;
    // A launch that computes A.x itself carries `rank` producer workgroups in front: the weight
    // workgroups leave them room, so that every workgroup of the launch is resident at once and no
    // weight wave has to wait for a producer that cannot start.
    const uint32_t max_waves = (256 * wg_per_cu - producers) * wg_waves;
    uint32_t rw = (n_wrows + max_waves - 1) / max_waves;
    if (even_rw && rw <= 4 && (rw & 1)) ++rw;
    uint32_t waves;
    p.persistent = rw > 4;
    if (rw <= 4) {
        // every wave resident, one chunk each
        waves = (n_wrows + rw - 1) / rw;
    } else {
        // more rows than one chunk per resident wave covers: a full grid of persistent waves that
        // walk several chunks.  Waves differ by at most one chunk, so the chunk height is the
        // largest (most loads in flight) that keeps that imbalance under 8 %.
        waves = max_waves;
        rw = even_rw ? 2 : 1;
        for (uint32_t cand = 4; cand > 1; cand -= even_rw ? 2 : 1) {
            const uint32_t most = (n_wrows + max_waves * cand - 1) / (max_waves * cand) * cand;  // rows of the busiest wave
            if (static_cast<uint64_t>(most) * max_waves * 100 <= static_cast<uint64_t>(n_wrows) * 108) {
                rw = cand;
                break;
            }
        }
    }
    uint32_t sg = slabs < 3 ? slabs : 3;
    while (rw * sg > 6) --sg;
    p.seg = seg;
    p.wg_waves = wg_waves;
    p.waves = waves;
    p.rw = rw;
    p.sg = sg;
    return p;
}

}  // namespace

}  // namespace lq4
