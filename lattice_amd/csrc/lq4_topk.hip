// Exact top-k selection over a vector of logits: the device side of the reference's two-stage
// lm_head top-k (shaders/qwen35.metal:1683-1778, 1868-1985).
//
// Small inputs take the reference's route: stage 1 sorts tiles of 1024 logits and keeps each
// tile's k best; merge passes then sort up to 2048 surviving candidates at a time and keep k,
// until one group is left.  Every pass is a full bitonic sort of its candidates, so each tile's
// list is its exact local top-k and the result is the first k entries of the globally sorted
// list — independent of tile size and fan-in.  Inputs of at least k blocks of 256 take the
// threshold route further down, which returns the same list without sorting.
// Ordering (qwen35.metal:1697-1703): higher logit first, ties to the lower token id; a NaN logit
// enters as the sentinel (-inf, 0xFFFFFFFF) and ranks last.
#include "lq4_internal.hpp"
#include "lq4_topk_dev.hpp"

namespace lq4 {

namespace {

// Descending bitonic sort of tg[0..N) by 256 threads.
template <int N>
__device__ __forceinline__ void bitonic_sort_desc(Cand* tg, uint32_t tid) {
    for (uint32_t step = 2; step <= N; step <<= 1) {
        for (uint32_t dist = step >> 1; dist > 0; dist >>= 1) {
            for (uint32_t idx = tid; idx < N; idx += 256) {
                const uint32_t ixj = idx ^ dist;
                if (ixj > idx) {
                    const Cand a = tg[idx], b = tg[ixj];
                    const bool swap = (idx & step) ? better(a, b) : better(b, a);
                    if (swap) {
                        tg[idx] = b;
                        tg[ixj] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

__device__ __forceinline__ void emit(const Cand* tg, uint32_t k, uint32_t group, uint32_t tid, Cand* out,
                                     float* out_logits, uint32_t* out_ids) {
    for (uint32_t o = tid; o < k; o += 256) {
        if (out_logits) {  // last pass: the caller's two arrays
            out_logits[o] = tg[o].logit;
            out_ids[o] = tg[o].id;
        } else {
            out[group * k + o] = tg[o];
        }
    }
}

constexpr uint32_t kTile = 1024;

__global__ __launch_bounds__(256) void topk_tile_kernel(const float* __restrict__ logits, uint32_t n, uint32_t k,
                                                        Cand* __restrict__ out, float* out_logits,
                                                        uint32_t* out_ids) {
    __shared__ Cand tg[kTile];
    const uint32_t tid = threadIdx.x;
    for (uint32_t slot = tid; slot < kTile; slot += 256) {
        const uint32_t i = blockIdx.x * kTile + slot;
        Cand c = sentinel();
        if (i < n) {
            const float v = logits[i];
            if (v == v) c = Cand{v, i};
        }
        tg[slot] = c;
    }
    __syncthreads();
    bitonic_sort_desc<kTile>(tg, tid);
    emit(tg, k, blockIdx.x, tid, out, out_logits, out_ids);
}

constexpr uint32_t kMergeSlots = 2048;

__global__ __launch_bounds__(256) void topk_merge_kernel(const Cand* __restrict__ in, uint32_t groups, uint32_t k,
                                                         uint32_t fan_in, Cand* __restrict__ out, float* out_logits,
                                                         uint32_t* out_ids) {
    __shared__ Cand tg[kMergeSlots];
    const uint32_t tid = threadIdx.x;
    const uint32_t first = blockIdx.x * fan_in;
    const uint32_t items = fan_in * k;  // <= kMergeSlots by construction
    for (uint32_t slot = tid; slot < kMergeSlots; slot += 256) {
        Cand c = sentinel();
        if (slot < items) {
            const uint32_t g = first + slot / k;
            if (g < groups) c = in[g * k + slot % k];
        }
        tg[slot] = c;
    }
    __syncthreads();
    bitonic_sort_desc<kMergeSlots>(tg, tid);
    emit(tg, k, blockIdx.x, tid, out, out_logits, out_ids);
}

// ---- fast path: threshold from block maxima, then rank the few survivors ---------------------
// The vector is cut into M <= 1024 blocks of `blk` logits.  tau = a key that at least k of the
// block maxima reach (the k-th best maximum, or a little below it).  At least k elements (those
// maxima) rank at or before tau, so every global top-k element does too, and only the blocks whose
// maximum reaches tau can contain such elements: at most topk_most_blocks(k) * blk survive.
// The survivors are ranked by counting, for each, how many survivors beat it: `better` is a
// strict total order, so ranks are distinct and rank r goes to output slot r.  No sorting, and
// the result is the same exact list the tile/merge path gives.
//
// For k <= 64 one launch does all of it.  Every wave reduces one block to its best key; the
// workgroup that draws the last ticket (all maxima are then in memory) finds tau, rescans the
// blocks whose maximum reaches tau (50 KB for k = 50) and ranks what it found.  The steps after
// the maxima are serial work for one workgroup, but each is short (a thousand keys, k blocks,
// typically 1-3 k survivors), and three launches with their ramp-up and drain are gone: 13.9 us
// instead of 17 for the top 50 of 248 320 logits.
//
// How the maxima reach the last workgroup: each is written with a device-scope atomic exchange,
// whose returned old value the wave waits for before its workgroup draws a ticket (another
// device-scope atomic); the last workgroup reads them with device-scope atomic loads.  Atomics at
// device scope are carried out where all compute dies see them, so a load issued after the last
// ticket came back finds every exchange done.  Plain stores with a device-wide fence before the
// ticket would be the textbook form; the fence writes the whole L2 back and, at one per
// workgroup, made the kernel 13 us slower.

// grid ceil(M / 4), block 256: wave w of workgroup g reduces block 4g + w of `blk` logits to its
// best key; the workgroup with the last ticket selects, rescans and ranks (see above).  `ticket`
// is zero between launches: the last workgroup puts it back.  `surv` holds topk_most_blocks(k) * blk
// candidates.
__global__ __launch_bounds__(256) void topk_select_kernel(const float* __restrict__ logits, uint32_t n, uint32_t blk,
                                                          uint32_t m, uint32_t k, uint64_t* maxima, Cand* surv,
                                                          uint32_t* ticket, float* __restrict__ out_logits,
                                                          uint32_t* __restrict__ out_ids) {
    __shared__ TopkTailShared ts;
    __shared__ uint32_t s_last;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    {
        const uint32_t b = blockIdx.x * 4 + (tid >> 6);
        if (b < m) {
            const uint32_t beg = b * blk;
            const uint32_t end = beg + blk < n ? beg + blk : n;
            uint64_t best = key_of(sentinel());
            for (uint32_t i = beg + lane; i < end; i += 64) {
                const uint64_t kk = key_of(load_cand(logits, i));
                best = kk > best ? kk : best;
            }
            best = wave_max_key(best);
            if (lane == 0) {
                // An exchange at device scope is carried out where every part of the chip sees it,
                // and once its old value has come back it is done: the empty statement below
                // takes that value, so the wave waits for it before the barrier and the ticket.
                // (A device-wide fence instead costs every workgroup a cache write-back.)
                const uint64_t old = __hip_atomic_exchange(maxima + b, best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                asm volatile("" ::"v"(static_cast<uint32_t>(old)));
            }
        }
    }
    __syncthreads();
    if (tid == 0) {
        const uint32_t t = atomicAdd(ticket, 1u);
        s_last = t == gridDim.x - 1;
        // every other workgroup has drawn: ready for the next launch
        if (s_last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!s_last) return;
    topk_select_tail<false>(logits, n, TopkBlocks{blk, 0, 1}, m, k, maxima, surv, ts, out_logits, out_ids);
}

// ---- the same selection as four launches, for large k ---------------------------------------
// The single kernel above leaves the rescan of the surviving blocks to one workgroup; from about
// 64 blocks on (k = 256: 320 KB of logits) a grid doing that work in parallel is faster even with
// three more launches: 20 us against 34 for k = 256 over 248 320 logits.

// grid M, block 256: key of the best candidate of block b of `blk` logits.
__global__ __launch_bounds__(256) void topk_blockmax_kernel(const float* __restrict__ logits, uint32_t n, uint32_t blk,
                                                            uint64_t* __restrict__ maxima) {
    __shared__ uint64_t part[4];
    const uint32_t beg = blockIdx.x * blk;
    const uint32_t end = beg + blk < n ? beg + blk : n;
    uint64_t best = key_of(sentinel());
    for (uint32_t i = beg + threadIdx.x; i < end; i += 256) {
        const uint64_t kk = key_of(load_cand(logits, i));
        best = kk > best ? kk : best;
    }
    best = wave_max_key(best);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w2 = 1; w2 < 4; ++w2) best = part[w2] > best ? part[w2] : best;
        maxima[blockIdx.x] = best;
    }
}

// grid ceil(M / 16), block 256: tau = k-th best of the M <= 1024 block maxima (equal keys, which
// only all-NaN blocks produce, are ordered by slot).  Workgroup 0 also clears the survivor counter
// and fills the output with sentinels (slots no survivor claims keep them).
__global__ __launch_bounds__(256) void topk_threshold_kernel(const uint64_t* __restrict__ maxima, uint32_t m, uint32_t k,
                                                             uint64_t* __restrict__ tau, uint32_t* __restrict__ counter,
                                                             float* __restrict__ out_logits,
                                                             uint32_t* __restrict__ out_ids) {
    __shared__ uint64_t s[1024];
    for (uint32_t i = threadIdx.x; i < 1024; i += 256) s[i] = i < m ? maxima[i] : 0ull;
    if (blockIdx.x == 0) {
        if (threadIdx.x == 0) *counter = 0;
        for (uint32_t o = threadIdx.x; o < k; o += 256) {
            out_logits[o] = -INFINITY;
            out_ids[o] = 0xFFFFFFFFu;
        }
    }
    __syncthreads();
    // 16 lanes per entry, each counting over every 16th slot.  Slots past m hold key 0, below
    // every real key.
    const uint32_t i = blockIdx.x * 16 + (threadIdx.x >> 4);
    const uint32_t sub = threadIdx.x & 15;
    const uint64_t c = s[i < m ? i : 0];
    uint32_t rank = 0;
    const uint32_t lim = (m + 15) & ~15u;
    for (uint32_t j = sub; j < lim; j += 16) {
        const uint64_t o = s[j];
        rank += (o > c) | ((o == c) & (j < i));
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) rank += __shfl_xor(rank, off, 64);
    if (i >= m || sub != 0) return;
    if (rank == k - 1) *tau = c;
}

constexpr uint32_t kCompactPerWg = 2048;

// Appends every element that ranks at or before tau to `surv` (order irrelevant).
__global__ __launch_bounds__(256) void topk_compact_kernel(const float* __restrict__ logits, uint32_t n,
                                                           const uint64_t* __restrict__ tau, Cand* __restrict__ surv,
                                                           uint32_t* __restrict__ counter) {
    const uint64_t t = *tau;
    const uint32_t beg = blockIdx.x * kCompactPerWg;
    const uint32_t end = beg + kCompactPerWg < n ? beg + kCompactPerWg : n;
    for (uint32_t i = beg + threadIdx.x; i < end; i += 256) {
        const Cand c = load_cand(logits, i);
        if (c.id != 0xFFFFFFFFu && key_of(c) >= t) surv[atomicAdd(counter, 1u)] = c;
    }
}

// Rank of each survivor = number of survivors that beat it; rank r < k goes to output slot r.
__global__ __launch_bounds__(256) void topk_rank_kernel(const Cand* __restrict__ surv, const uint32_t* __restrict__ counter,
                                                        uint32_t k, float* __restrict__ out_logits,
                                                        uint32_t* __restrict__ out_ids) {
    __shared__ uint64_t s[1024];
    const uint32_t total = *counter;
    const uint32_t rounds = (total + gridDim.x * 256 - 1) / (gridDim.x * 256);
    for (uint32_t r = 0; r < rounds; ++r) {
        const uint32_t i = (r * gridDim.x + blockIdx.x) * 256 + threadIdx.x;
        const Cand c = i < total ? surv[i] : sentinel();
        const uint64_t ck = key_of(c);
        uint32_t rank = 0;
        for (uint32_t base = 0; base < total; base += 1024) {
            __syncthreads();
            for (uint32_t j = threadIdx.x; j < 1024; j += 256) s[j] = base + j < total ? key_of(surv[base + j]) : 0ull;
            __syncthreads();
            const uint32_t lim = total - base < 1024 ? (total - base + 15) & ~15u : 1024;
            for (uint32_t j0 = 0; j0 < lim; j0 += 16) {  // slots past `total` hold key 0
#pragma unroll
                for (uint32_t u = 0; u < 16; ++u) rank += s[j0 + u] > ck;
            }
        }
        if (i < total && rank < k) {
            out_logits[rank] = c.logit;
            out_ids[rank] = c.id;
        }
    }
}

// blocks of `blk` logits such that there are at most 1024 of them; 0 = fast path not applicable
uint32_t fast_block(uint32_t n, uint32_t k) {
    uint32_t blk = 64;  // a wave's width; smaller blocks only add maxima
    while ((n + blk - 1) / blk > 1024) blk <<= 1;
    return (n + blk - 1) / blk >= k ? blk : 0;
}

}  // namespace

size_t topk_scratch_bytes(uint32_t n, uint32_t k) {
    const uint32_t blk = fast_block(n, k);
    if (blk)  // maxima[1024] | tau, counter (large k only) | survivors
        return (1024 + 2) * sizeof(uint64_t) + static_cast<size_t>(topk_most_blocks(k)) * blk * sizeof(Cand);
    const size_t tiles = (n + kTile - 1) / kTile;
    return 2 * tiles * k * sizeof(Cand);  // two candidate buffers, ping-pong
}

void launch_topk(const float* logits, uint32_t n, uint32_t k, void* scratch, uint32_t* ticket, float* out_logits,
                 uint32_t* out_ids, hipStream_t stream) {
    if (const uint32_t blk = fast_block(n, k)) {
        const uint32_t m = (n + blk - 1) / blk;
        uint64_t* maxima = static_cast<uint64_t*>(scratch);
        Cand* surv = reinterpret_cast<Cand*>(maxima + 1024);
        if (k <= kSingleKernelMaxK) {
            hipLaunchKernelGGL(topk_select_kernel, dim3((m + 3) / 4), dim3(256), 0, stream, logits, n, blk, m, k,
                               maxima, surv, ticket, out_logits, out_ids);
            return;
        }
        uint64_t* tau = maxima + 1024;
        uint32_t* counter = reinterpret_cast<uint32_t*>(tau + 1);
        surv = reinterpret_cast<Cand*>(tau + 2);
        hipLaunchKernelGGL(topk_blockmax_kernel, dim3(m), dim3(256), 0, stream, logits, n, blk, maxima);
        hipLaunchKernelGGL(topk_threshold_kernel, dim3((m + 15) / 16), dim3(256), 0, stream, maxima, m, k, tau, counter,
                           out_logits, out_ids);
        hipLaunchKernelGGL(topk_compact_kernel, dim3((n + kCompactPerWg - 1) / kCompactPerWg), dim3(256), 0, stream,
                           logits, n, tau, surv, counter);
        hipLaunchKernelGGL(topk_rank_kernel, dim3(64), dim3(256), 0, stream, surv, counter, k, out_logits, out_ids);
        return;
    }
    uint32_t groups = (n + kTile - 1) / kTile;
    Cand* a = static_cast<Cand*>(scratch);
    Cand* b = a + static_cast<size_t>(groups) * k;
    const bool single = groups == 1;
    hipLaunchKernelGGL(topk_tile_kernel, dim3(groups), dim3(256), 0, stream, logits, n, k, a,
                       single ? out_logits : nullptr, single ? out_ids : nullptr);
    while (groups > 1) {
        uint32_t fan_in = kMergeSlots / k;
        fan_in = fan_in < groups ? fan_in : groups;
        const uint32_t out_groups = (groups + fan_in - 1) / fan_in;
        const bool last = out_groups == 1;
        hipLaunchKernelGGL(topk_merge_kernel, dim3(out_groups), dim3(256), 0, stream, a, groups, k, fan_in, b,
                           last ? out_logits : nullptr, last ? out_ids : nullptr);
        Cand* t = a;
        a = b;
        b = t;
        groups = out_groups;
    }
}

}  // namespace lq4
