// Grouped expert GEMV of the MoE path on the integer matrix cores.
//
// One workgroup handles one expert, one chunk of that expert's output rows and up to four of the (token, slot) pairs
// routed to it ("a pass"; an expert more tokens chose is served in several), in the arithmetic of lq4_gemv_i8.hip's
// "wide" form: v_mfma_i32_16x16x32_i8
// multiplies one Q4 block (K = 32) of 16 weight rows with 16 activation columns.  The activations of a pair are
// staged as fixed point scaled per block (x = xs * q, |q| < 2^22) and cut into three signed byte digits, operand row
// 4 * pair + digit, so four pairs fill the operand; the block's scale and bias are applied to the integer sums in f32.
// Lane l receives, for weight row l % 16, the three digit sums of pair l / 16: no value crosses lanes after the
// instruction.  Per instruction (320 bytes of weights): two masks to spread the nibbles, two conversions of the block
// header, about eight operations to join the digits and update the sum, against about forty for the same bytes in the
// 4x4x4 f16 form this file replaced, which was bound by exactly that instruction count.
//
// GATE_UP = true: a wave's tiles come in twos, gate rows [r, r + 16) and up rows [I + r, I + r + 16) of the expert
// ([E, 2I, H], gate rows first: crates/inference/src/model/qwen35/moe.rs:127-190); the lane that owns (row, pair) in
// one owns it in the other and writes h[pair, row] = silu(g) * u.  GATE_UP = false: plain rows of the down
// projection ([E, H, I]), o[pair, row] = W . h[pair].
//
// Memory: a unit is 16 rows x 8 blocks (2.5 KB); lane l loads block l % 8 of rows l / 8 and l / 8 + 8 as whole 20-byte
// blocks, and passes them through a wave-private LDS tile into the operand layout (the next unit on its way meanwhile).
// CW waves split the 8-block chunks of a tile and add their partial sums through LDS in wave order; TW = 8 / CW tiles
// are worked on side by side; a workgroup does `rounds` such rounds.
//
// Grid.  The y index counts only the (expert, pass) combinations that exist, found from the routing table itself (up
// to 512 pairs, a thread per pair: moe_combo_from_ids) or from the grouping tables of a launch before this one
// (moe_combo_from_tables): a workgroup that finds nothing to do still holds a CU slot for a microsecond, and a grid
// over every expert and every possible pass is mostly such workgroups.
//
// What the time stamps of a development build showed for 16 tokens of top 8 among 64 experts (73 MB gate/up, 37 MB
// down), and what this file does about it: (1) with four waves and 32 output rows a workgroup, 912 workgroups had
// work and 768 fit the chip: the last 144 started when the first ended, 14 us into a 25 us launch -- eight waves over
// 64 (gate/up) or 256 (down) rows make about 460, which all start at once; (2) a CU's share of the memory system is
// about 18 KB/us and answers in the order of asking, so activations asked for behind a ring of four units of every
// wave on the CU arrived last, and the matrix work that could have run beside the stream ran after it -- a wave
// holds one unit (kDepth); (3) per CU the vector instructions (about 130 a unit) and the LDS traffic (14 KB a unit)
// each still add up to about a third of the streaming time.
//
// Precision: weights and integer sums are exact; an activation is rounded to a multiple of its block's largest
// magnitude / 4194000 (1.2e-7 of the block maximum, the resolution of the f32 activation itself).  A block whose
// largest magnitude is below 2^-100 counts as zero; an infinite or NaN activation makes the outputs of its pair NaN.
#include "lq4_internal.hpp"

namespace lq4 {

namespace {

constexpr int kMoePassPairs = 4;  // pairs a workgroup serves in one pass over its rows

struct MoeGemvArgs {
    const uint8_t* w;        // expert-major Q4 tensor
    const float* x;          // activation rows
    float* out;              // h (GATE_UP) or o
    const int32_t* offsets;  // [E + 1]
    const int32_t* order;    // pair indices grouped by expert
    const int32_t* ids;      // routed expert of every pair; not null = find the expert's pairs here instead of in
    uint32_t n_pairs;        // offsets/order (up to 512 pairs: saves a launch and two dependent loads)
    uint32_t rows_per_expert;  // weight rows of one expert (2I or H)
    uint32_t out_rows;         // output rows per pair (I or H)
    uint32_t k;                // reduction length (H or I)
    uint32_t x_stride;         // floats between activation rows
    uint32_t x_div;            // activation row of a pair = pair / x_div (top_k for x, 1 for h)
    uint32_t rounds;           // rounds of tiles per workgroup
    const uint8_t* w_last;     // not null: the last expert lives here, not behind the others in w
    uint32_t experts;          // experts in all
};

// The grid's y index counts (expert, pass) combinations that exist, not every expert times every possible pass: a
// workgroup with nothing to do still holds a CU slot for a microsecond, and a grid over all of them is mostly such
// workgroups (16 tokens of top 8 among 64 experts make about 60 combinations, not 64 x 4).  The host bounds their
// number (combo_bound); a workgroup whose y is beyond the real count exits.
//
// From the grouping tables of a launch before this one (offsets [experts + 1], order [pairs]): combination blockIdx.y
// in expert order (see expert_at); its pairs into s_pair[0 .. n), in the tables' (stable) order.  Returns n (0: beyond the
// combinations; the same value in every thread) and the expert.  s_cnt holds a word per wave, s_misc two.
template <int THREADS>
__device__ __forceinline__ int moe_combo_from_tables(const MoeGemvArgs& p, int32_t* s_pair, int32_t* s_cnt,
                                                     int32_t* s_misc, uint32_t& e) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Order: expert order, except that an expert with tensors of its own (w_last: one that every token chose, all
    // its passes full-length work) comes first instead of forming the tail of the launch.
    auto expert_at = [&](uint32_t i) { return p.w_last == nullptr ? i : i == 0 ? p.experts - 1 : i - 1; };
    auto passes_at = [&](uint32_t i) {
        if (i >= p.experts) return 0;
        const uint32_t ee = expert_at(i);
        return (p.offsets[ee + 1] - p.offsets[ee] + kMoePassPairs - 1) / kMoePassPairs;
    };
    // a thread takes `per` consecutive places of the order; combinations before its first = an exclusive scan
    const uint32_t per = (p.experts + THREADS - 1) / THREADS, e0 = static_cast<uint32_t>(tid) * per;
    int local = 0;
    for (uint32_t r = 0; r < per; ++r) local += passes_at(e0 + r);
    int incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
    }
    if (lane == 63) s_cnt[wave] = incl;
    __syncthreads();
    int before = 0, n_combos = 0;
#pragma unroll
    for (int w2 = 0; w2 < THREADS / 64; ++w2) {
        before += w2 < wave ? s_cnt[w2] : 0;
        n_combos += s_cnt[w2];
    }
    const int y = static_cast<int>(blockIdx.y);
    if (y >= n_combos) return 0;
    int c = before + incl - local;
    if (y >= c && y < c + local) {  // one thread: the combination is among its experts
        for (uint32_t r = 0; r < per; ++r) {
            const int n = passes_at(e0 + r);
            if (y < c + n) {
                s_misc[0] = static_cast<int32_t>(expert_at(e0 + r));
                s_misc[1] = y - c;
                break;
            }
            c += n;
        }
    }
    __syncthreads();
    e = static_cast<uint32_t>(s_misc[0]);
    const int32_t beg = p.offsets[e] + s_misc[1] * kMoePassPairs, end = p.offsets[e + 1];
    const int nt = end - beg < kMoePassPairs ? end - beg : kMoePassPairs;
    if (tid < nt) s_pair[tid] = p.order[beg + tid];
    __syncthreads();
    return nt;
}

// From the routing table itself (ids; a thread per pair: n_pairs <= THREADS): combination blockIdx.y in the order of
// the combinations' first pairs; no grouping launch, no offsets -> order -> row chain of dependent loads.
//   `mask` is LDS for experts x THREADS / 64 64-bit words (bit t % 64 of word t / 64 of an expert = pair t chose it;
//   set with atomic ORs, so the table does not depend on the order of arrival), free again on return; s_misc holds 4
//   words, s_cnt one per wave.
// Returns n (0: blockIdx.y is beyond the combinations) and the expert.  An id outside [0, experts) matches nothing.
template <int THREADS>
__device__ __forceinline__ int moe_combo_from_ids(const MoeGemvArgs& p, unsigned long long* mask, int32_t* s_pair,
                                               int32_t* s_cnt, int32_t* s_misc, uint32_t& e) {
    constexpr int W = THREADS / 64;  // words of an expert's row in the table
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int32_t id = static_cast<uint32_t>(tid) < p.n_pairs ? p.ids[tid] : -1;
    for (uint32_t i = tid; i < p.experts * W; i += THREADS) mask[i] = 0ull;
    const bool mine = static_cast<uint32_t>(id) < p.experts;
    if (!mine) id = 0;
    __syncthreads();
    if (mine) __hip_atomic_fetch_or(&mask[id * W + wave], 1ull << lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();
    // rank of this pair among the pairs of its expert, and how many there are
    int rank = 0, total = 0;
#pragma unroll
    for (int w2 = 0; w2 < W; ++w2) {
        const unsigned long long m = mask[id * W + w2];
        total += __popcll(m);
        rank += w2 < wave ? __popcll(m) : w2 == wave ? __popcll(m & ((1ull << lane) - 1ull)) : 0;
    }
    // every fourth pair of an expert opens a combination; its index = such pairs before it
    const bool leader = mine && (rank & 3) == 0;
    const uint64_t lmask = __ballot(leader);
    if (lane == 0) s_cnt[wave] = __popcll(lmask);
    __syncthreads();  // (also: every read of the table is done)
    int before = 0, n_combos = 0;
#pragma unroll
    for (int w2 = 0; w2 < THREADS / 64; ++w2) {
        before += w2 < wave ? s_cnt[w2] : 0;
        n_combos += s_cnt[w2];
    }
    if (static_cast<int>(blockIdx.y) >= n_combos) return 0;
    if (leader && before + __popcll(lmask & ((1ull << lane) - 1ull)) == static_cast<int>(blockIdx.y)) {
        s_misc[0] = id;
        s_misc[1] = rank;
        s_misc[2] = total - rank < kMoePassPairs ? total - rank : kMoePassPairs;
    }
    __syncthreads();
    e = static_cast<uint32_t>(s_misc[0]);
    const int r0 = s_misc[1], nt = s_misc[2];
    if (mine && static_cast<uint32_t>(id) == e && rank >= r0 && rank < r0 + kMoePassPairs) s_pair[rank - r0] = tid;
    __syncthreads();
    return nt;
}

typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kBpw = 8;            // blocks per chunk
constexpr int kTilePitch = 44;     // dwords per row of the LDS tile (40 used; 44 r mod 64 differs for every r < 16)
constexpr int kTileDwords = 16 * kTilePitch;
constexpr int kXqBytes = 512;      // per block: [4 k groups][16 operand rows] x 8 bytes
constexpr int kXfBytes = 64;       // per block: [4 pairs]{xs, xs * sum of the block's fixed-point x, -, -} f32
// Units a wave holds in registers (beside the one in its LDS tile).  One: the next unit is requested when the current
// one has been copied into the tile and arrives while that is multiplied.  Deeper rings were measured and are
// slower (16 tokens of top 8 among 64 experts, both launches and the combine: 4 / 3 / 2 / 1 units 36.2 / 35.7 / 34.7 /
// 34.2 us; 64 tokens 74.3 / 69.7 / 68.3 / 67.2): the 3600 waves of a launch with one unit each have about what the
// memory system holds in flight anyway (9 MB), and whatever is asked for beyond that only queues in front of the
// loads a workgroup's start waits for (the routing table, the activations).
constexpr int kDepth = 1;
constexpr float kQScale = 4194000.0f;

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

__device__ __forceinline__ float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float half_lo(uint32_t sb) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(sb & 0xFFFFu)));
}
__device__ __forceinline__ float half_hi(uint32_t sb) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(sb >> 16)));
}
__device__ __forceinline__ float silu(float v) { return v * (1.0f / (1.0f + expf(-v))); }

size_t lds_bytes(uint32_t nb, uint32_t waves) {
    const uint32_t nbp = (nb + kBpw - 1) / kBpw * kBpw;  // whole chunks
    return static_cast<size_t>(nb) * kXqBytes + static_cast<size_t>(nbp) * kXfBytes + static_cast<size_t>(waves) * kTileDwords * 4 +
           static_cast<size_t>(waves) * 64 * 2 * 4;
}

// p.rounds = rounds of the workgroup; the launcher gives every wave a chunk (chunks of a row >= CW).
// Grid (row chunks, a bound on the (expert, pass) combinations).  FROM_IDS: these come from the routing table, else
// from the grouping tables.
template <bool GATE_UP, int CW, int TW, bool FROM_IDS>
__global__ __launch_bounds__(64 * CW * TW) void moe_expert_i8(MoeGemvArgs p) {
    constexpr int kWaves = CW * TW, kThreads = 64 * kWaves;
    constexpr uint32_t TPR = GATE_UP ? 2 : 1;  // tiles of a wave per round
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __shared__ int32_t s_pair[kMoePassPairs];
    __shared__ int32_t s_cnt[kWaves];
    __shared__ int32_t s_misc[4];
    uint32_t e;
    int nt;
    if constexpr (FROM_IDS) nt = moe_combo_from_ids<kThreads>(p, reinterpret_cast<unsigned long long*>(smem), s_pair, s_cnt, s_misc, e);
    else nt = moe_combo_from_tables<kThreads>(p, s_pair, s_cnt, s_misc, e);
    if (nt == 0) return;

    const uint32_t tw = wave / CW, cw = wave % CW;
    const uint32_t nb = p.k / kBlockWeights;
    const uint32_t row_bytes = nb * static_cast<uint32_t>(kBlockBytes);
    const uint32_t chunks = (nb + kBpw - 1) / kBpw;
    const uint32_t my_chunks = cw < chunks ? (chunks - cw + CW - 1) / CW : 0;  // chunk c * CW + cw
    const uint32_t rounds = p.rounds;
    const uint32_t units = rounds * TPR * my_chunks;  // unit u = (tile u / my_chunks, chunk u % my_chunks)
    auto first_row = [&](uint32_t rd) { return ((blockIdx.x * rounds + rd) * TW + tw) * 16; };  // output row

    // LDS: [nb] activation digits | [whole chunks] activation scales and sums, zero beyond the row's last block |
    // [waves] tiles | [waves][64][2] partial sums
    const uint32_t nbp = chunks * kBpw;
    uint8_t* const xq = smem;
    uint8_t* const xf = xq + static_cast<size_t>(nb) * kXqBytes;
    uint32_t* const tile = reinterpret_cast<uint32_t*>(xf + static_cast<size_t>(nbp) * kXfBytes) + wave * kTileDwords;
    float* const part = reinterpret_cast<float*>(xf + static_cast<size_t>(nbp) * kXfBytes) + kWaves * kTileDwords;

    const uint8_t* const wbase = (p.w_last != nullptr && e == p.experts - 1)
                                     ? p.w_last
                                     : p.w + static_cast<size_t>(e) * p.rows_per_expert * row_bytes;

    // load mapping: lane = (block jl, row rq), rows rq and rq + 8 of the tile
    const uint32_t jl = lane % kBpw, rq = lane / kBpw;
    auto load_unit = [&](Q4BlockRaw (&buf)[2], uint32_t u) {
        const uint32_t ti = u / my_chunks, c = u - ti * my_chunks;
        const uint32_t rd = ti / TPR, which = ti - rd * TPR;
        const uint32_t row0 = first_row(rd);
        uint32_t blk = (c * CW + cw) * kBpw + jl;
        if (blk >= nb) blk = nb - 1;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t row = row0 + rq + 8 * i;
            if (row >= p.out_rows) row = p.out_rows - 1;
            if (GATE_UP && which) row += p.out_rows;
            const uint8_t* bp = wbase + static_cast<size_t>(row) * row_bytes + blk * static_cast<uint32_t>(kBlockBytes);
            buf[i].sb = *reinterpret_cast<const uint32_t*>(bp);
            typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));
            const u32x4u q = *reinterpret_cast<const u32x4u*>(bp + 4);
            buf[i].q[0] = q.x; buf[i].q[1] = q.y; buf[i].q[2] = q.z; buf[i].q[3] = q.w;
        }
    };

    // ---- stage the activations of the pass: task = (pair, block, k group), 8 values each ----------------------
    const uint32_t items = nb * 4;                              // tasks of one pair
    const uint32_t n_tasks = static_cast<uint32_t>(nt) * items;  // (whole quads: a multiple of 4)
    const float* xrow[kMoePassPairs];
#pragma unroll
    for (int b = 0; b < kMoePassPairs; ++b) {
        const int32_t pair = s_pair[b < nt ? b : 0];
        xrow[b] = p.x + static_cast<size_t>(static_cast<uint32_t>(pair) / p.x_div) * p.x_stride;
    }
    auto task_of = [&](uint32_t idx, uint32_t& b, uint32_t& blk, uint32_t& kg) {
        b = (idx >= items ? 1u : 0u) + (idx >= 2 * items ? 1u : 0u) + (idx >= 3 * items ? 1u : 0u);
        const uint32_t rem = idx - b * items;
        blk = rem >> 2;
        kg = rem & 3;
    };
    auto task_ptr = [&](uint32_t idx) {
        uint32_t b, blk, kg;
        task_of(idx < n_tasks ? idx : 0, b, blk, kg);  // a task that does not exist re-reads the first one
        const float* xr = b == 0 ? xrow[0] : b == 1 ? xrow[1] : b == 2 ? xrow[2] : xrow[3];
        return reinterpret_cast<const float4*>(xr + blk * kBlockWeights + kg * 8);
    };
    auto quad_max = [](uint32_t v) {
        v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false)));
        return max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false)));
    };
    auto quad_sum = [](int v) {
        v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);
        return v + __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);
    };
    // (called by whole quads of lanes: the four k groups of one (pair, block))
    auto stage_task = [&](uint32_t idx, const float4 xa, const float4 xb) {
        uint32_t b, blk, kg;
        task_of(idx, b, blk, kg);
        const float v[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        // largest magnitude as a bit pattern: infinities and NaNs come out on top of every finite value
        uint32_t abits = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) abits = max(abits, as_u32(v[i]) & 0x7FFFFFFFu);
        abits = quad_max(abits);
        const bool finite = abits < 0x7F800000u;
        float inv = 0.0f, xs = 0.0f;
        if (finite && abits >= 0x0D800000u) {  // 2^-100 and up
            xs = as_f32(abits) * (1.0f / kQScale);
            inv = __builtin_amdgcn_rcpf(xs);
        } else if (!finite) {
            xs = as_f32(0x7FC00000u);
        }
        // 1.5 * 2^23 + q as a float has q in its low 23 bits in two's complement: bits = 0x4B400000 + q
        uint32_t qb[8], sum_bits = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            qb[i] = as_u32(fmaf(v[i], inv, 12582912.0f));
            sum_bits += qb[i];
        }
        const int sum = quad_sum(static_cast<int>(sum_bits - 8u * 0x4B400000u));
        // Digits -128..127 from the lowest up: byte 0 of q, byte 1 of q + 0x80, byte 2 of q + 0x8080 (minus the
        // 0x40 the float's own bits hold there).  Byte i of an operand word pair = element {0, 2, 4, 6, 1, 3, 5,
        // 7}[i] of the k group: the order in which the two masks lay out a payload dword's nibbles.
        uint32_t dg[3][2];
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            const uint32_t add = t == 0 ? 0u : t == 1 ? 0x80u : 0xFFC08080u;
            const uint32_t sel_lo = 0x0c0c0400u + 0x0101u * t, sel_hi = 0x04000c0cu + 0x01010000u * t;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t e0 = qb[h] + add, e1 = qb[2 + h] + add, e2 = qb[4 + h] + add, e3 = qb[6 + h] + add;
                dg[t][h] = __builtin_amdgcn_perm(e1, e0, sel_lo) | __builtin_amdgcn_perm(e3, e2, sel_hi);
            }
        }
        // operand rows 4 b .. 4 b + 2: the highest digit first; row 4 b + 3 is never read back
        uint2* dst = reinterpret_cast<uint2*>(xq + static_cast<size_t>(blk) * kXqBytes + kg * 128 + (4 * b) * 8);
#pragma unroll
        for (int t = 0; t < 3; ++t) dst[t] = make_uint2(dg[2 - t][0], dg[2 - t][1]);
        dst[3] = make_uint2(0u, 0u);
        if (kg == 0) {
            float* f = reinterpret_cast<float*>(xf + static_cast<size_t>(blk) * kXfBytes);
            f[4 * b] = xs;
            f[4 * b + 1] = xs * static_cast<float>(sum);
        }
    };

    // The values of a thread's first tasks are requested before any weight (loads are answered in the order a CU
    // issued them: behind the weight prefetch the staging would wait for the weights), all at once.
    constexpr int kHoist = kWaves >= 8 ? 2 : 4;  // (K = 2048 with four pairs: all of them)
    float4 xv[kHoist][2];
#pragma unroll
    for (int it = 0; it < kHoist; ++it) {
        const float4* xp = task_ptr(tid + it * kThreads);
        xv[it][0] = xp[0];
        xv[it][1] = xp[1];
    }
    Q4BlockRaw ring[kDepth][2];
#pragma unroll
    for (int i = 0; i < kDepth; ++i) {
        if (static_cast<uint32_t>(i) < units) load_unit(ring[i], i);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads
#pragma unroll
    for (int it = 0; it < kHoist; ++it) {
        const uint32_t idx = tid + it * kThreads;
        if (idx < n_tasks) stage_task(idx, xv[it][0], xv[it][1]);
    }
    for (uint32_t idx = tid + kHoist * kThreads; idx < n_tasks; idx += kThreads) {
        const float4* xp = task_ptr(idx);
        stage_task(idx, xp[0], xp[1]);
    }
    // (pairs the pass does not have: their operand rows and scales hold whatever LDS held, and their results are dropped)
    // blocks past the end of a row (K not a whole number of chunks): scale and sum zero, so they count for nothing
    for (uint32_t i = nb * 16 + tid; i < nbp * 16; i += kThreads) reinterpret_cast<float*>(xf)[i] = 0.0f;
    __syncthreads();

    // ---- the product ----
    const uint32_t r = lane & 15, g = lane >> 4;  // operand mapping: weight row r of the tile, k group / pair g
    const int32_t my_pair = s_pair[static_cast<int>(g) < nt ? g : 0];
    float acc[2] = {0.0f, 0.0f};  // GATE_UP: gate, up
    auto process = [&](Q4BlockRaw (&cur)[2], uint32_t u) {
        if (u >= units) return;  // uniform
        // through the tile: tile[row][5 * block + d]; the buffer is then free for the unit kDepth ahead
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t* tp = tile + (rq + 8 * i) * kTilePitch + 5 * jl;
            tp[0] = cur[i].sb;
            tp[1] = cur[i].q[0]; tp[2] = cur[i].q[1]; tp[3] = cur[i].q[2]; tp[4] = cur[i].q[3];
        }
        if (u + kDepth < units) load_unit(cur, u + kDepth);  // uniform
        const uint32_t ti = u / my_chunks, c = u - ti * my_chunks;
        const uint32_t rd = ti / TPR, which = ti - rd * TPR;
        const uint32_t blk0 = (c * CW + cw) * kBpw;
        const uint32_t* tr = tile + r * kTilePitch;
        float sum = 0.0f;
        // four blocks at a time, straight-line: their LDS reads, then their four matrix instructions back to back,
        // then their results (a block past the end of the row re-reads the row's last one and meets zero scales)
#pragma unroll
        for (int j0 = 0; j0 < kBpw; j0 += 4) {
            uint32_t sb[4], qd[4];
            long aop[4];
            float2 f[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const uint32_t blk_raw = blk0 + j0 + jj;
                const uint32_t blk = blk_raw < nb ? blk_raw : nb - 1;  // uniform
                sb[jj] = tr[5 * (j0 + jj)];
                qd[jj] = tr[5 * (j0 + jj) + 1 + g];
                aop[jj] = *reinterpret_cast<const long*>(xq + static_cast<size_t>(blk) * kXqBytes + lane * 8);
                f[jj] = *reinterpret_cast<const float2*>(xf + static_cast<size_t>(blk_raw) * kXfBytes + g * 16);
            }
            int4v d[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const uint32_t even = qd[jj] & 0x0F0F0F0Fu, odd = (qd[jj] >> 4) & 0x0F0F0F0Fu;
                const long bop = static_cast<long>((static_cast<uint64_t>(odd) << 32) | even);
                const int4v zero = {0, 0, 0, 0};
                d[jj] = __builtin_amdgcn_mfma_i32_16x16x32_i8(aop[jj], bop, zero, 0, 0, 0);
            }
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const float scale = half_lo(sb[jj]), bias = half_hi(sb[jj]);
                // the top digit's sum times 2^16 is exact in f32, so is 256 mid + low: one rounding in the add
                const float d0 = fmaf(static_cast<float>(d[jj].x), 65536.0f, static_cast<float>(d[jj].y * 256 + d[jj].z));
                sum = fmaf(scale * f[jj].x, d0, sum);
                sum = fmaf(bias, f[jj].y, sum);
            }
        }
        if (GATE_UP && which) acc[1] += sum;  // uniform
        else acc[0] += sum;
        if (c + 1 == my_chunks && which + 1 == TPR) {  // the wave's part of the round is complete (uniform)
            if constexpr (CW > 1) {
                __syncthreads();  // (every wave passes here once a round)
                part[(wave * 64 + lane) * 2] = acc[0];
                part[(wave * 64 + lane) * 2 + 1] = acc[1];
                __syncthreads();
                acc[0] = 0.0f;
                acc[1] = 0.0f;
                if (cw == 0) {
#pragma unroll
                    for (int v = 0; v < CW; ++v) {
                        acc[0] += part[((tw * CW + v) * 64 + lane) * 2];
                        acc[1] += part[((tw * CW + v) * 64 + lane) * 2 + 1];
                    }
                }
            }
            const uint32_t row = first_row(rd) + r;
            if (cw == 0 && static_cast<int>(g) < nt && row < p.out_rows)
                p.out[static_cast<size_t>(my_pair) * p.out_rows + row] = GATE_UP ? silu(acc[0]) * acc[1] : acc[0];
            acc[0] = 0.0f;
            acc[1] = 0.0f;
        }
    };
    for (uint32_t u = 0; u < units; u += kDepth) {
#pragma unroll
        for (int i = 0; i < kDepth; ++i) process(ring[i], u + i);
    }
}

template <bool GATE_UP, int CW, int TW, bool FROM_IDS>
void launch_cw(const MoeGemvArgs& a, uint32_t rows_per_wg, uint32_t passes, size_t lds, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(moe_expert_i8<GATE_UP, CW, TW, FROM_IDS>), 159 * 1024);  // the rest is static
    const uint32_t row_chunks = (a.out_rows + rows_per_wg - 1) / rows_per_wg;
    // combinations at most: all but the last of an expert hold four pairs (pairs / 4 + experts); every one has a
    // first pair of its own (pairs); experts x passes
    uint32_t combo_bound = a.n_pairs / kMoePassPairs + a.experts;
    if (combo_bound > a.n_pairs) combo_bound = a.n_pairs;
    if (combo_bound > a.experts * passes) combo_bound = a.experts * passes;
    hipLaunchKernelGGL((moe_expert_i8<GATE_UP, CW, TW, FROM_IDS>), dim3(row_chunks, combo_bound), dim3(64 * CW * TW), lds,
                       stream, a);
}

template <bool GATE_UP, int CW, int TW>
void launch_from(bool from_ids, const MoeGemvArgs& a, uint32_t rows_per_wg, uint32_t passes, size_t lds, hipStream_t stream) {
    if (from_ids) launch_cw<GATE_UP, CW, TW, true>(a, rows_per_wg, passes, lds, stream);
    else launch_cw<GATE_UP, CW, TW, false>(a, rows_per_wg, passes, lds, stream);
}

}  // namespace

// The matrix-core form serves reductions whose staged activations fit its LDS.
bool moe_i8_serves(uint32_t k) { return k >= kBlockWeights && lds_bytes(k / kBlockWeights, 8) <= 150 * 1024; }

namespace {

template <bool GATE_UP>
void launch_moe_expert_i8(MoeGemvArgs a, uint32_t num_experts, uint32_t max_pairs_per_expert, hipStream_t stream) {
    constexpr uint32_t kWaves = 8;
    const uint32_t nb = a.k / kBlockWeights;
    size_t lds = lds_bytes(nb, kWaves);
    if (!moe_i8_serves(a.k)) return;  // the caller asked first
    a.experts = num_experts;
    const bool from_ids = a.ids != nullptr;  // (the caller: up to kMoeIdsMaxPairs pairs and kMoeIdsMaxExperts experts)
    if (from_ids && lds < static_cast<size_t>(num_experts) * kWaves * 8) lds = static_cast<size_t>(num_experts) * kWaves * 8;
    // Waves split K only where every one of them finds a chunk or two.  Workgroups of eight waves over about 64
    // (gate/up) or 256 (down) output rows, 160 KB of blocks each: 16 tokens of top 8 among 64 experts then make
    // about 460 workgroups with work, which all start at once (two fit a CU).  Measured there against four waves
    // and 32 / 128 rows (912 workgroups, three or seven a CU): 40.3 -> 37.3 us for the two launches and the
    // combine; with four waves the last 144 of the gate/up workgroups started when the first ones ended.
    const uint32_t chunks = (nb + kBpw - 1) / kBpw;
    const uint32_t cw = chunks >= 4 ? 2 : 1, tw = kWaves / cw;
    const uint32_t target_rows = GATE_UP ? 64 : 256;
    uint32_t rounds = target_rows / (tw * 16);
    if (rounds < 1) rounds = 1;
    a.rounds = rounds;
    const uint32_t rows_per_wg = rounds * tw * 16, passes = (max_pairs_per_expert + kMoePassPairs - 1) / kMoePassPairs;
    if (cw == 2) launch_from<GATE_UP, 2, 4>(from_ids, a, rows_per_wg, passes, lds, stream);
    else launch_from<GATE_UP, 1, 8>(from_ids, a, rows_per_wg, passes, lds, stream);
}

}  // namespace

void launch_moe_gate_up_i8(const uint8_t* gate_up, uint32_t num_experts, uint32_t inter, uint32_t hidden, const float* x,
                           uint32_t tokens, uint32_t top_k, const int32_t* offsets, const int32_t* order,
                           const int32_t* ids, float* h, hipStream_t stream, const uint8_t* last_expert) {
    MoeGemvArgs a{gate_up, x, h, offsets, order, ids, tokens * top_k, 2 * inter, inter, hidden, hidden, top_k, 0,
                  last_expert, num_experts};
    launch_moe_expert_i8<true>(a, num_experts, tokens, stream);
}

void launch_moe_down_i8(const uint8_t* down, uint32_t num_experts, uint32_t inter, uint32_t hidden, const float* h,
                        uint32_t tokens, uint32_t top_k, const int32_t* offsets, const int32_t* order,
                        const int32_t* ids, float* o, hipStream_t stream, const uint8_t* last_expert) {
    MoeGemvArgs a{down, h, o, offsets, order, ids, tokens * top_k, hidden, hidden, inter, inter, 1, 0, last_expert,
                  num_experts};
    launch_moe_expert_i8<false>(a, num_experts, tokens, stream);
}

}  // namespace lq4
