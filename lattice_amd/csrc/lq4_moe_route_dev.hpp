// The router of one token, by one wave (shared by the stand-alone routing kernel and by the decode-sized
// MoE kernel that routes inside its own launch).
#pragma once
#include "lq4_internal.hpp"

namespace lq4 {

// Wave-wide maximum / minimum of a 32-bit unsigned value, in every lane: row steps with
// data-parallel-primitive moves, then the two row-swap instructions across the four rows.
template <bool MAX>
__device__ __forceinline__ uint32_t wave_extreme(uint32_t v) {
    auto pick = [](uint32_t a, uint32_t b) { return MAX ? (a > b ? a : b) : (a < b ? a : b); };
    v = pick(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false)));
    v = pick(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false)));
    v = pick(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, false)));
    v = pick(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, false)));
    uint32_t a = v, b = v;
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    v = pick(a, b);
    a = v;
    b = v;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return pick(a, b);
}

// Router of one token by one whole wave (crates/inference/src/model/qwen35/moe.rs:80-125 semantics: softmax
// over all experts, the top_k largest probabilities in rank order with the lower expert id first
// among equals, renormalised).  Lane l holds experts l, l + 64, ...; the exponentials are computed
// in parallel, their sum is taken in expert order from LDS (the order a sequential loop uses, so
// the probabilities are the same bits), and every rank is one wave-wide maximum of the probability
// bits followed by a wave-wide minimum of the expert ids that reach it.
// kPerLane: experts per lane, 64 * kPerLane >= num_experts.  `s_ev`: 64 * kPerLane floats of LDS that
// only this wave touches.  Lane r < top_k returns rank r's expert id (-1: fewer experts than ranks) and
// renormalised weight.
template <int kPerLane>
__device__ __forceinline__ void route_one_token(const float* __restrict__ lg, uint32_t num_experts, uint32_t top_k,
                                                uint32_t lane, float* s_ev, int32_t& out_id, float& out_w) {
    float v[kPerLane];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const uint32_t e = 64u * i + lane;
        v[i] = e < num_experts ? lg[e] : -INFINITY;
        if (v[i] > mx) mx = v[i];  // a NaN operand is ignored (f32::max semantics)
    }
    {   // wave maximum of floats that are never NaN: order-preserving integer keys
        const uint32_t bits = __builtin_bit_cast(uint32_t, mx);
        const uint32_t key = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
        const uint32_t best = wave_extreme<true>(key);
        mx = __builtin_bit_cast(float, (best & 0x80000000u) ? (best & 0x7fffffffu) : ~best);
    }
    const bool finite_max = fabsf(mx) != INFINITY;
    float ev[kPerLane];
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const uint32_t e = 64u * i + lane;
        ev[i] = finite_max && e < num_experts ? expf(v[i] - mx) : 0.0f;
        if (e < num_experts) s_ev[e] = ev[i];
    }
    // one wave wrote, the same wave reads: its LDS operations are carried out in program order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float denom = 0.0f;
    if (finite_max)
        for (uint32_t e = 0; e < num_experts; ++e) denom += s_ev[e];  // every lane, same order, same sum
    const bool live = finite_max && denom > 0.0f;
    // probabilities as orderable bits (they are >= 0 or, not live, all zero); 0xFFFFFFFF marks
    // "no expert here" below every real one once inverted... taken experts drop to key 0
    uint32_t key[kPerLane];
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const uint32_t e = 64u * i + lane;
        const float p = live ? ev[i] / denom : 0.0f;
        key[i] = e < num_experts ? __builtin_bit_cast(uint32_t, p) + 1u : 0u;  // + 1: a real expert beats "none"
    }
    int32_t my_id = -1;
    float my_p = -INFINITY;
    for (uint32_t r = 0; r < top_k; ++r) {
        uint32_t best_key = 0u, best_i = 0u;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i)
            if (key[i] > best_key) {  // strict: the lower expert id of equals
                best_key = key[i];
                best_i = i;
            }
        const uint32_t top = wave_extreme<true>(best_key);
        if (top == 0u) break;  // fewer experts than ranks: the remaining ranks stay (-1, -inf)
        const uint32_t cand = best_key == top ? 64u * best_i + lane : 0xFFFFFFFFu;
        const uint32_t win = wave_extreme<false>(cand);
        if (cand == win) {
#pragma unroll
            for (int i = 0; i < kPerLane; ++i)
                if (static_cast<uint32_t>(i) == best_i) key[i] = 0u;
        }
        if (lane == r) {
            my_id = static_cast<int32_t>(win);
            my_p = __builtin_bit_cast(float, top - 1u);
        }
    }
    float top_sum = 0.0f;
    for (uint32_t r = 0; r < top_k; ++r)
        top_sum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_p), static_cast<int>(r)));
    out_id = my_id;
    out_w = top_sum > 0.0f ? my_p / top_sum : my_p;
}

}  // namespace lq4
