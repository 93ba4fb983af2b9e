// Device-side pieces of the exact top-k selection that more than one kernel uses: the candidate
// order (shaders/qwen35.metal:1697-1703: higher logit first, ties to the lower token id, NaN last as
// the (-inf, 0xFFFFFFFF) sentinel), its 64-bit key, the radix select, and the selection tail that one
// workgroup runs once every block maximum is known (used by the stand-alone top-k kernel and by the
// lm_head GEMV that selects in its own launch).
#pragma once
#include <type_traits>

#include "lq4_internal.hpp"

namespace lq4 {

typedef float float4v __attribute__((ext_vector_type(4)));

struct Cand {
    float logit;
    uint32_t id;
};

__device__ __forceinline__ Cand sentinel() { return Cand{-INFINITY, 0xFFFFFFFFu}; }

__device__ __forceinline__ bool better(Cand a, Cand b) {
    if (a.logit != a.logit) return false;
    if (b.logit != b.logit) return true;
    if (a.logit != b.logit) return a.logit > b.logit;
    return a.id < b.id;
}

// 64-bit sort key of a candidate: a ranks before b  <=>  key(a) > key(b).  High word: the logit's
// bits mapped to an unsigned order (-0 counted as +0, as the float comparison does); low word:
// ~id, so ties go to the lower id.  NaN never gets here (it became the sentinel, the lowest key).
__device__ __forceinline__ uint64_t key_of(Cand c) {
    uint32_t u = __float_as_uint(c.logit);
    if (c.logit == 0.0f) u = 0;
    u ^= (u >> 31) ? 0xFFFFFFFFu : 0x80000000u;
    return (static_cast<uint64_t>(u) << 32) | static_cast<uint32_t>(~c.id);
}

__device__ __forceinline__ Cand load_cand(const float* logits, uint32_t i) {
    const float v = logits[i];
    return v == v ? Cand{v, i} : sentinel();
}

__device__ __forceinline__ uint64_t wave_max_key(uint64_t k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const uint32_t lo = __shfl_xor(static_cast<uint32_t>(k), off, 64);
        const uint32_t hi = __shfl_xor(static_cast<uint32_t>(k >> 32), off, 64);
        const uint64_t o = (static_cast<uint64_t>(hi) << 32) | lo;
        k = o > k ? o : k;
    }
    return k;
}

// A candidate this workgroup stored a moment ago, read back past the vector cache.
__device__ __forceinline__ Cand load_survivor(const Cand* surv, uint32_t i) {
    const uint64_t raw =
        __hip_atomic_load(reinterpret_cast<const uint64_t*>(surv) + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return Cand{__uint_as_float(static_cast<uint32_t>(raw)), static_cast<uint32_t>(raw >> 32)};
}

struct SelectShared {
    uint32_t hist[256];
    uint64_t prefix;
    uint32_t need;
};

// The k-th largest (k >= 1, counted with multiplicity) of the `count` >= k keys get(0..count):
// eight rounds of an 8-bit radix select, most significant digit first.  A round counts the digit
// of every key that still matches the digits fixed so far; wave 0 walks the 256 counts from the
// top to the digit that holds the `need`-th key.  Called by all 256 threads of the workgroup.
template <typename Get>
__device__ __forceinline__ uint64_t select_kth_key(Get get, uint32_t count, uint32_t k, SelectShared& sh) {
    const uint32_t tid = threadIdx.x;
    uint64_t prefix = 0;
    uint32_t need = k;
    for (int shift = 56; shift >= 0; shift -= 8) {
        sh.hist[tid] = 0;
        __syncthreads();
        for (uint32_t i = tid; i < count; i += 256) {
            const uint64_t key = get(i);
            // (x >> 1) >> 63-or-less: a shift by 64 is not defined, the first round matches all
            const bool match = (((key ^ prefix) >> 1) >> (shift + 7)) == 0;
            if (match) atomicAdd(&sh.hist[(key >> shift) & 255], 1u);
        }
        __syncthreads();
        if (tid < 64) {  // lane l owns digits 255 - 4l .. 252 - 4l, highest first
            uint32_t c[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) c[j] = sh.hist[255 - 4 * tid - j];
            const uint32_t sum = (c[0] + c[1]) + (c[2] + c[3]);
            uint32_t incl = sum;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const uint32_t t = __shfl_up(incl, off, 64);
                if (tid >= static_cast<uint32_t>(off)) incl += t;
            }
            uint32_t run = incl - sum;
            if (run < need && need <= incl) {  // exactly one lane: the counts above it fall short
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (run < need && need <= run + c[j]) {
                        sh.prefix = prefix | (static_cast<uint64_t>(255 - 4 * tid - j) << shift);
                        sh.need = need - run;
                    }
                    run += c[j];
                }
            }
        }
        __syncthreads();
        prefix = sh.prefix;
        need = sh.need;
    }
    return prefix;
}

constexpr uint32_t kRankSlots = 1024;  // survivors ranked out of LDS
constexpr uint32_t kSingleKernelMaxK = 64;
constexpr int kGatherUnits = 16;       // 16-byte loads a thread has in flight when rescanning: 50 blocks of 256 in one go

// The threshold may let up to this many blocks through instead of exactly k: it is found in fewer
// steps, and the survivor buffer is sized for it.
__host__ __device__ constexpr uint32_t topk_most_blocks(uint32_t k) { return k + (k >> 2) + 4; }


// How the logits are cut into the blocks whose maxima steer the selection.  Block b is `runs` runs of
// `run` consecutive logits (a multiple of 4), run r starting at r * stride + b * run.  Contiguous
// blocks of `blk` logits: {blk, 0, 1}.  The rows a GEMV workgroup of W waves x R side-by-side rows
// produces: {W * R, waves of the launch * R, wave-rows per wave}.
struct TopkBlocks {
    uint32_t run, stride, runs;
};

// LDS of the selection tail (19.6 KB).
struct TopkTailShared {
    uint64_t keys[kRankSlots];
    float vals[kRankSlots];
    uint32_t ids[kRankSlots];
    uint16_t sel[1024];
    SelectShared sh;
    uint32_t cnt[2][4];
    uint32_t count, nsel, tail;
};

// A logit that reaches tau's value becomes a survivor: ranked out of LDS while the slots last, in
// memory beyond them.  One compare, which NaN fails; an element that ties tau's logit with a higher id
// passes although it ranks after tau, which costs a slot and nothing else.
__device__ __forceinline__ void topk_keep_one(TopkTailShared& ts, Cand* surv, float v, uint32_t i, float tau_f) {
    if (!(v >= tau_f)) return;
    const uint32_t slot = atomicAdd(&ts.count, 1u);
    if (slot < kRankSlots) {  // the usual case stays in LDS: no store to wait for before the ranking
        ts.vals[slot] = v;
        ts.ids[slot] = i;
    } else {
        surv[slot - kRankSlots] = Cand{v, i};
    }
}

// The exact top k of `n` logits, given the best key of each of the m <= 1024 blocks (m >= k), by one
// workgroup of 256 threads (every thread calls; barriers inside).  tau = a key that at least k of the
// block maxima reach (the k-th best maximum, or a little below it).  At least k elements (those
// maxima) rank at or before tau, so every global top-k element does too, and only the blocks whose
// maximum reaches tau can contain such elements: at most topk_most_blocks(k) blocks survive.  The
// survivors are ranked by counting, for each, how many survivors beat it: `better` is a strict total
// order, so ranks are distinct and rank r goes to output slot r.
// COHERENT: logits and maxima were written earlier in this same launch by other workgroups (logits
// with device-scope stores that the writers waited for): they are read with device-scope loads, which
// go past this compute die's caches.  Otherwise the logits come from an earlier launch and are read
// with plain loads, 16 bytes at a time where alignment allows.
// `surv` holds topk_most_blocks(k) * runs * run candidates (those that do not fit the LDS slots go there).
template <bool COHERENT>
__device__ __forceinline__ void topk_select_tail(const float* __restrict__ logits, uint32_t n, TopkBlocks bl, uint32_t m,
                                                 uint32_t k, const uint64_t* maxima, Cand* surv, TopkTailShared& ts,
                                                 float* __restrict__ out_logits, uint32_t* __restrict__ out_ids) {
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    if (tid == 0) {
        ts.count = 0;
        ts.nsel = 0;
        ts.tail = 0;
    }
    for (uint32_t o = tid; o < k; o += 256) {  // slots no survivor claims (NaN input) keep the sentinel
        out_logits[o] = -INFINITY;
        out_ids[o] = 0xFFFFFFFFu;
    }

    // tau: a key that at least k and at most `most` of the block maxima reach.  Built from the top
    // bit down (a bit stays set if k maxima still reach the result); the first value that no more
    // than `most` maxima reach will do, and if none comes up the loop ends at the k-th best
    // maximum itself.  A step is four compares per thread and one barrier.
    uint64_t kk[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)  // device-scope loads, as the maxima were written; 0: below every key
        kk[j] = tid + 256 * j < m ? __hip_atomic_load(maxima + tid + 256 * j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                  : 0ull;
    const uint32_t most = topk_most_blocks(k);
    uint64_t tau = 0;
    for (int bit = 63, par = 0; bit >= 0; --bit, par ^= 1) {
        const uint64_t cand = tau | (1ull << bit);
        uint32_t c = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) c += __popcll(__ballot(kk[j] >= cand));
        if (lane == 0) ts.cnt[par][tid >> 6] = c;
        __syncthreads();  // one barrier a step: the two halves of cnt take turns
        c = (ts.cnt[par][0] + ts.cnt[par][1]) + (ts.cnt[par][2] + ts.cnt[par][3]);
        if (c >= k) {
            tau = cand;
            if (c <= most) break;
        }
    }

    // (the block that holds the vector's last logit: its odd end is read separately below)
    const uint32_t last_blk = bl.runs == 1 ? (n - 1) / bl.run : ((n - 1) % bl.stride) / bl.run;
    // the blocks that can hold an element at or before tau: at most `most` (more only if tau is
    // the all-NaN key, and then the extra blocks hold nothing that passes the test below)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (kk[j] >= tau && tid + 256 * j < m) {
            ts.sel[atomicAdd(&ts.nsel, 1u)] = static_cast<uint16_t>(tid + 256 * j);
            if (tid + 256 * j == last_blk) ts.tail = 1;
        }
    }
    __syncthreads();
    const uint32_t nsel = ts.nsel;
    // Survivors: every logit of those blocks that is not below tau's logit (tau's high word mapped
    // back to a float; a word below every real key means that -inf still passes).  One compare,
    // which NaN fails; an element that ties tau's logit with a higher id passes although it ranks
    // after tau, which costs a slot and nothing else.
    const uint32_t tau_u = static_cast<uint32_t>(tau >> 32);
    const float tau_f = tau_u < 0x007FFFFFu ? -INFINITY
                                            : __uint_as_float((tau_u >> 31) ? tau_u ^ 0x80000000u : ~tau_u);
    // All loads of a batch are issued before the first is looked at: one workgroup has to cover the
    // latency of the selected blocks by itself.  It also runs this code once per launch, straight from
    // memory: the batch is as small as the number of units allows (G loads per thread in flight), a unit
    // none of whose four logits reaches tau (nearly all of them) costs four compares and a branch, and
    // the rest is kept out of line, so that the whole phase is a few hundred instructions.
    const bool vec = COHERENT || (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
    // COHERENT: 16-byte loads that go past this compute die's caches (the device-scope cache policy on a
    // buffer load; bytes past the end of the buffer read as zero).  The logits buffer is 16-byte aligned.
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(logits), 0,
                                                                      static_cast<int>(n * sizeof(float)), 0x00020000);
    constexpr int kDeviceScope = 16;  // sc1
    const uint32_t upr = bl.run >> 2;          // 16-byte units per run
    const uint32_t upb = upr * bl.runs;        // ... per block
    const uint32_t units = nsel * upb;
    // u / d for the small u and d of this loop as one multiplication: inv = ceil(2^32 / d) is exact for
    // u * d < 2^32 (d = 1 would need 2^32 itself and is tested for)
    const uint32_t inv_upb = 0xFFFFFFFFu / upb + 1, inv_upr = 0xFFFFFFFFu / upr + 1;
    auto first_of = [&](uint32_t u) {  // index of the first logit of unit u (n: none)
        const uint32_t s = upb == 1 ? u : __umulhi(u, inv_upb), q = u - s * upb;
        const uint32_t r = upr == 1 ? q : __umulhi(q, inv_upr), within = q - r * upr;
        // 64-bit: a run index past the logits' end (the last runs of the later blocks) may not wrap
        const uint64_t i64 = static_cast<uint64_t>(r) * bl.stride + static_cast<uint64_t>(ts.sel[s]) * bl.run + 4 * within;
        return i64 < n ? static_cast<uint32_t>(i64) : n;
    };
    auto gather = [&](auto g_tag) {
        constexpr int G = decltype(g_tag)::value;
        for (uint32_t u0 = 0; u0 < units; u0 += 256 * G) {
            float4v v[G];
            uint32_t idx[G];
#pragma unroll
            for (int j = 0; j < G; ++j) {
                const uint32_t u = u0 + j * 256 + tid;
                const uint32_t i = u < units ? first_of(u) : n;
                idx[j] = i;
                if constexpr (COHERENT) {
                    v[j] = __builtin_bit_cast(float4v, __builtin_amdgcn_raw_buffer_load_b128(
                                                           rsrc, static_cast<int>(i * sizeof(float)), 0, kDeviceScope));
                } else {
                    v[j] = *reinterpret_cast<const float4v*>(logits + (i + 4 <= n ? i : 0));
                }
            }
#pragma unroll
            for (int j = 0; j < G; ++j) {
                // logits past the end (of the vector, or of the last whole unit when read in place) do not count
                const uint32_t left = COHERENT ? n - idx[j] : (idx[j] + 4 <= n ? 4u : 0u);
                const bool hit = ((v[j][0] >= tau_f) & (left > 0)) | ((v[j][1] >= tau_f) & (left > 1)) |
                                 ((v[j][2] >= tau_f) & (left > 2)) | ((v[j][3] >= tau_f) & (left > 3));
                if (hit) {
#pragma unroll
                    for (uint32_t e = 0; e < 4; ++e)
                        if (e < left) topk_keep_one(ts, surv, v[j][e], idx[j] + e, tau_f);
                }
            }
        }
    };
    if (vec) {
        if (units <= 256 * 2) gather(std::integral_constant<int, 2>{});
        else gather(std::integral_constant<int, kGatherUnits>{});
        if constexpr (!COHERENT) {
            // the logits after the last whole unit of the vector, if their block was selected
            const uint32_t whole = n & ~3u;
            if (tid < (n & 3) && ts.tail) topk_keep_one(ts, surv, logits[whole + tid], whole + tid, tau_f);
        }
    } else {
        // logits that are not 16-byte aligned: one at a time
        for (uint32_t e = tid; e < units * 4; e += 256) {
            const uint32_t i = first_of(e >> 2) + (e & 3);
            if (i < n) topk_keep_one(ts, surv, logits[i], i, tau_f);
        }
    }
    __syncthreads();
    uint32_t total = ts.count;
    for (uint32_t e = tid; e < (total < kRankSlots ? total : kRankSlots); e += 256)
        ts.keys[e] = key_of(Cand{ts.vals[e], ts.ids[e]});
    if (total > kRankSlots) {
        // too many to rank from LDS (sorted or constant input): keep exactly the k best of them; the
        // ones beyond the LDS slots are read back from memory
        __threadfence();
        __syncthreads();
        auto key_at = [&](uint32_t i) { return i < kRankSlots ? ts.keys[i] : key_of(load_survivor(surv, i - kRankSlots)); };
        const uint64_t tau2 = select_kth_key(key_at, total, k, ts.sh);
        // the k keepers are gathered in the (now free) histogram before they replace the first slots
        uint64_t* keep_keys = reinterpret_cast<uint64_t*>(ts.sh.hist);          // [k <= 64]
        float* keep_vals = reinterpret_cast<float*>(ts.sh.hist + 2 * kSingleKernelMaxK);
        if (tid == 0) ts.count = 0;
        __syncthreads();
        for (uint32_t i = tid; i < total; i += 256) {
            const uint64_t key = key_at(i);
            if (key >= tau2) {  // keys are distinct: k of them
                const uint32_t slot = atomicAdd(&ts.count, 1u);
                keep_keys[slot] = key;
                keep_vals[slot] = i < kRankSlots ? ts.vals[i] : load_survivor(surv, i - kRankSlots).logit;
            }
        }
        __syncthreads();
        total = ts.count;
        if (tid < total) {
            ts.keys[tid] = keep_keys[tid];
            ts.vals[tid] = keep_vals[tid];
        }
        __syncthreads();
    }
    const uint32_t lim = (total + 15) & ~15u;
    for (uint32_t i = total + tid; i < lim; i += 256) ts.keys[i] = 0;  // below every real key
    __syncthreads();
    for (uint32_t e = tid; e < total; e += 256) {
        const uint64_t ck = ts.keys[e];
        uint32_t rank = 0;
        for (uint32_t j0 = 0; j0 < lim; j0 += 16) {
#pragma unroll
            for (uint32_t u = 0; u < 16; ++u) rank += ts.keys[j0 + u] > ck;
        }
        if (rank < k) {
            out_logits[rank] = ts.vals[e];
            out_ids[rank] = ~static_cast<uint32_t>(ck);
        }
    }
}

}  // namespace lq4
