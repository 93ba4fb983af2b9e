// Few-token prefill GEMM: Y[M,N] = X[M,K] . W[N,K]^T for 2 .. 128 tokens, over Q4, Q8_0 or Q3 blocks.
//
// With so few tokens the product is bound by streaming W once, like the decode GEMV, but there
// are too many tokens for the 4x4x4 GEMV kernel and too few to fill the 128-token tiles of the
// prefill kernels.  Two launches:
//
// 1. pack_x: the activations are converted to f16 once and laid out exactly as the matrix-core
//    B operand wants them: for K step s (128 wide), token group t (16 tokens) and instruction j,
//    the 64 lanes' 16-byte operands are contiguous (1 KB).  Lane (c = lane % 16, g = lane / 16)
//    holds token 16 t + c, K offsets 128 s + 32 g + 8 j .. + 7 in the order x0 x4 x1 x5 x2 x6 x3
//    x7 (the order in which the Q4 dequantiser emits a packed dword; memory order for the sibling
//    formats).  Tokens past M and K past the end are zero-filled, so the main kernel needs no tail
//    handling on this operand.
//
// 2. gemm_q4_skinny<RT, FMT, NTG>: a workgroup of eight waves owns 16 RT weight rows against a tile
//    of NTG groups of 16 tokens.  Wave w takes K steps w, w + 8, ...; per step it loads its own Q4 blocks
//    (lane (r, g) owns block g of row r of the step, as in the large prefill kernel) and the
//    packed operands with fully coalesced 16-byte loads, dequantises in registers and issues
//    v_mfma_f32_16x16x32_f16.  No LDS staging and no barrier in the K loop: nothing is shared
//    between waves.  Two steps are in flight per wave; every load is unconditional (a load behind a
//    run-time condition would make the compiler wait for loads it cannot count).
//    Each wave adds its share of the LoRA delta (ranks w, w + 8, ...) to its partial result in
//    f32; the eight partial results then meet in LDS in a fixed order and y is stored once.
//    LA = true (Q4, rank <= 16): the factor t = A . X of the workgroup's token tile is computed here as well, A
//    riding through the K loop as one more 16-row tile against the same packed operands (f16 inputs, f32
//    accumulation, like the product itself), so that no launch for t precedes this one.  Every workgroup repeats
//    it for its token tile: 64 KB of A from L2 beside the 256 KB of packed X it reads anyway.
//
// Dequantised value: half(q*d + b) with one rounding (shaders/gemm_q4_tiled.metal:57-66), f32
// accumulation.
#include "lq4_internal.hpp"

namespace lq4 {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kWavesK = 8;   // waves of a workgroup, each a K slice
constexpr int kTokens = 64;  // tokens per workgroup: four groups of 16
constexpr int TK = 128;      // K per step: four Q4 blocks

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

struct U4 {
    uint32_t v[4];
};

__device__ __forceinline__ half2v as_h2(uint32_t v) { return __builtin_bit_cast(half2v, v); }
__device__ __forceinline__ uint32_t as_u32(half2v v) { return __builtin_bit_cast(uint32_t, v); }

// One packed dword (weights 8j..8j+7) -> f16 weights in the order w0 w4 w1 w5 w2 w6 w3 w7.  A
// masked dword OR-ed into the mantissa of 1024.0 (or 64.0) is the pair (1024+n_lo, 1024+n_hi);
// a packed subtract makes it (n_lo, n_hi) exactly, a packed fma applies scale and bias.
__device__ __forceinline__ U4 dequant8(uint32_t q, half2v d2, half2v b2) {
    const half2v k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
    const half2v k64 = {static_cast<_Float16>(64.0f), static_cast<_Float16>(64.0f)};
    const uint32_t q8 = q >> 8;
    const half2v t0 = as_h2((q & 0x000F000Fu) | 0x64006400u) - k1024;
    const half2v t1 = as_h2((q & 0x00F000F0u) | 0x54005400u) - k64;
    const half2v t2 = as_h2((q8 & 0x000F000Fu) | 0x64006400u) - k1024;
    const half2v t3 = as_h2((q8 & 0x00F000F0u) | 0x54005400u) - k64;
    U4 out;
    out.v[0] = as_u32(__builtin_elementwise_fma(t0, d2, b2));
    out.v[1] = as_u32(__builtin_elementwise_fma(t1, d2, b2));
    out.v[2] = as_u32(__builtin_elementwise_fma(t2, d2, b2));
    out.v[3] = as_u32(__builtin_elementwise_fma(t3, d2, b2));
    return out;
}

// Sibling formats (FMT 1 = Q8_0, 2 = Q3): their decoders emit the eight weights of an instruction
// in memory order, so their activations are packed without the interleave.
struct __attribute__((packed, aligned(2))) Q8BlockRaw {
    uint16_t d;
    uint32_t q[8];  // weight i in byte i
};
struct __attribute__((packed, aligned(4))) Q3BlockRaw {
    uint32_t sb;
    uint32_t lo[2];  // weight i of 16-weight half h at bits 2i of lo[h]
    uint32_t hi;     // weight i at bit i
};
template <int FMT>
struct WBlockOf {
    typedef Q4BlockRaw type;
    static constexpr uint32_t kBytes = 20;
};
template <>
struct WBlockOf<1> {
    typedef Q8BlockRaw type;
    static constexpr uint32_t kBytes = 34;
};
template <>
struct WBlockOf<2> {
    typedef Q3BlockRaw type;
    static constexpr uint32_t kBytes = 16;
};

// Q8_0: two packed dwords (weights 8j..8j+7) -> half(q * d).  A sign-flipped byte (q + 128) under the
// exponent byte of 1024.0 is 1024 + 128 + q exactly; subtract, then one multiply with one rounding.
__device__ __forceinline__ U4 dequant8_q8(uint32_t qa, uint32_t qb, half2v d2) {
    const half2v k1152 = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    const uint32_t ua = qa ^ 0x80808080u, ub = qb ^ 0x80808080u;
    U4 out;
    out.v[0] = as_u32((as_h2(__builtin_amdgcn_perm(0x64646464u, ua, 0x04010400u)) - k1152) * d2);
    out.v[1] = as_u32((as_h2(__builtin_amdgcn_perm(0x64646464u, ua, 0x04030402u)) - k1152) * d2);
    out.v[2] = as_u32((as_h2(__builtin_amdgcn_perm(0x64646464u, ub, 0x04010400u)) - k1152) * d2);
    out.v[3] = as_u32((as_h2(__builtin_amdgcn_perm(0x64646464u, ub, 0x04030402u)) - k1152) * d2);
    return out;
}

// Q3: weights 8j..8j+7 -> half(q * d + b), q = low2 | hi << 2.
__device__ __forceinline__ U4 dequant8_q3(const Q3BlockRaw& b, int j, half2v d2, half2v b2) {
    const half2v k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
    const uint32_t lw = (b.lo[j >> 1] >> (16 * (j & 1))) & 0xffffu;  // 8 two-bit fields
    const uint32_t hw = (b.hi >> (8 * j)) & 0xffu;                   // 8 bits
    U4 out;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t l4 = lw >> (4 * p), h2 = hw >> (2 * p);
        const uint32_t qa = (l4 & 3u) | ((h2 & 1u) << 2);
        const uint32_t qb = ((l4 >> 2) & 3u) | ((h2 & 2u) << 1);
        out.v[p] = as_u32(__builtin_elementwise_fma(as_h2(0x64006400u | qa | (qb << 16)) - k1024, d2, b2));
    }
    return out;
}

__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {
    const half2v h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return as_u32(h);
}

__device__ __forceinline__ float load_b(const void* b, int is_f16, size_t idx) {
    return is_f16 ? static_cast<float>(static_cast<const _Float16*>(b)[idx]) : static_cast<const float*>(b)[idx];
}

// grid (K steps, token groups), 256 threads = 4 instructions x 64 lanes of one (step, group).
// INTERLEAVE: the x0 x4 x1 x5 .. order of the Q4 decoder; false = memory order (sibling formats).
template <bool X_F16, bool INTERLEAVE>
__global__ __launch_bounds__(256) void pack_x_kernel(const void* __restrict__ xv, uint32_t m, uint32_t k,
                                                     uint4* __restrict__ xp) {
    const uint32_t s = blockIdx.x, t = blockIdx.y, groups = gridDim.y;
    const int j = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t token = 16 * t + (lane & 15);
    const uint32_t koff = s * TK + 32 * (lane >> 4) + 8 * j;
    uint4 out = make_uint4(0, 0, 0, 0);
    if (token < m && koff < k) {
        if (X_F16) {
            const uint4 c = *reinterpret_cast<const uint4*>(static_cast<const _Float16*>(xv) +
                                                            static_cast<size_t>(token) * k + koff);
            if (INTERLEAVE) {
                out.x = __builtin_amdgcn_perm(c.z, c.x, 0x05040100u);  // x0..x7 -> x0 x4 x1 x5 x2 x6 x3 x7
                out.y = __builtin_amdgcn_perm(c.z, c.x, 0x07060302u);
                out.z = __builtin_amdgcn_perm(c.w, c.y, 0x05040100u);
                out.w = __builtin_amdgcn_perm(c.w, c.y, 0x07060302u);
            } else {
                out = c;
            }
        } else {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) +
                                                              static_cast<size_t>(token) * k + koff);
            const float4 lo = p[0], hi = p[1];
            if (INTERLEAVE) {
                out.x = pack_h2(lo.x, hi.x);
                out.y = pack_h2(lo.y, hi.y);
                out.z = pack_h2(lo.z, hi.z);
                out.w = pack_h2(lo.w, hi.w);
            } else {
                out.x = pack_h2(lo.x, lo.y);
                out.y = pack_h2(lo.z, lo.w);
                out.z = pack_h2(hi.x, hi.y);
                out.w = pack_h2(hi.z, hi.w);
            }
        }
    }
    xp[((static_cast<size_t>(s) * groups + t) * 4 + j) * 64 + lane] = out;
}

// RT: 16-row weight tiles per wave (rows per workgroup = 16 RT).  grid (ceil(N / 16 RT), token tiles).
// FMT: 0 = Q4, 1 = Q8_0, 2 = Q3 blocks.
// NTG: 16-token groups a workgroup computes (1, 2 or 4); a token tile with fewer groups re-reads its
// last group and drops the results.  tile_groups (<= NTG): token groups from one workgroup's tile to the next
// (grid.y tiles: four groups a tile, or two where NTG is held at two for a larger batch).  Fixed per instantiation, like the prefetches of the K loop below:
// a load behind a run-time condition makes the compiler wait for loads it cannot count, and the
// pipeline collapses to one unit in flight.
// LA: lora.a is the adapter's A packed by gemm_skinny_pack_lora_a and t = A . X is computed here (rank <= 16, Q4
// only); lora.t is then not read.
template <int RT, int FMT, int NTG, bool LA = false>
__global__ __launch_bounds__(64 * kWavesK) void gemm_q4_skinny(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                                const uint4* __restrict__ xp, uint32_t m,
                                                                float* __restrict__ y, LoraEpilogue lora,
                                                                uint32_t tile_groups) {
    static_assert(!LA || FMT == 0, "the adapter's A is packed in the Q4 decoder's order");
    static_assert(!LA || NTG <= 2, "with A in the K loop four token groups do not fit the registers");
    extern __shared__ float4v red[];  // 4 slots of RT * NTG * 64 accumulators; LA: then 8 * NTG * 64 partial t, then t

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15;
    const int g = lane >> 4;

    const uint32_t n0 = blockIdx.x * (16 * RT);
    const uint32_t groups = (m + 15) / 16;             // token groups in X (and in the packed image)
    const uint32_t tg0 = blockIdx.y * tile_groups;  // first token group of this workgroup
    const uint32_t ntg = groups - tg0 < tile_groups ? groups - tg0 : tile_groups;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t steps_total = (nb + 3) / 4;
    const uint32_t cnt = steps_total > static_cast<uint32_t>(wave) ? (steps_total - wave + kWavesK - 1) / kWavesK : 0;

    typedef typename WBlockOf<FMT>::type WBlock;
    constexpr uint32_t kBytes = WBlockOf<FMT>::kBytes;
    const uint8_t* w_row[RT];
#pragma unroll
    for (int u = 0; u < RT; ++u) {
        uint32_t row = n0 + 16 * u + lr;
        row = row < n ? row : n - 1;
        w_row[u] = w + static_cast<size_t>(row) * (nb * kBytes);
    }

    // LA: A packed like the activations (lq4_pack_lora_a): the operands of step s, instruction j at [(4 s + j) * 64 + lane]
    const uint4* const a_lane = static_cast<const uint4*>(lora.a) + lane;
    // The LoRA factor B of this wave's first two ranks (w and w + 8) is requested now, as raw bits, and converted in
    // the epilogue: requested there, the loads' whole latency stood between the K loop and the reduction (two token
    // groups of K steps a wave on a 2048-long row: the launch is latency from end to end).
    // (one row tile only: with two, the sixteen registers this holds through the K loop spill)
    constexpr bool kEarlyB = RT == 1;
    uint32_t b_raw[2][RT][4];
    if (kEarlyB && lora.rank) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const uint32_t jj = wave + p * kWavesK;
            const uint32_t jc = jj < lora.rank ? jj : 0;
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    uint32_t row = n0 + 16 * r + 4 * g + v;
                    row = row < n ? row : n - 1;
                    const size_t idx = static_cast<size_t>(row) * lora.rank + jc;
                    b_raw[p][r][v] = lora.b_is_f16 ? static_cast<uint32_t>(static_cast<const uint16_t*>(lora.b)[idx])
                                                   : static_cast<const uint32_t*>(lora.b)[idx];
                }
        }
    }
    struct Unit {
        WBlock wb[RT];
        uint4 x[NTG][4];  // [token group][instruction]
        uint4 a[LA ? 4 : 1];  // LA: the lane's operand of A for instruction j
    };
    uint32_t xg[NTG];  // packed-image group of token group t (clamped to the last one)
#pragma unroll
    for (int t = 0; t < NTG; ++t) xg[t] = tg0 + t < groups ? tg0 + t : groups - 1;
    // i-th step of this wave
    auto load = [&](Unit& u, uint32_t i) {
        const uint32_t s = wave + i * kWavesK;
        uint32_t blk = s * 4 + g;
        blk = blk < nb ? blk : nb - 1;
#pragma unroll
        for (int r = 0; r < RT; ++r) u.wb[r] = *reinterpret_cast<const WBlock*>(w_row[r] + blk * kBytes);
        if constexpr (LA) {
            const uint32_t sc = s < steps_total ? s : steps_total - 1;  // (a wave's clamped re-read of its last step)
#pragma unroll
            for (int j = 0; j < 4; ++j) u.a[j] = a_lane[(static_cast<size_t>(sc) * 4 + j) * 64];
        }
        const uint4* xs = xp + static_cast<size_t>(s) * groups * 256 + lane;
#pragma unroll
        for (int t = 0; t < NTG; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) u.x[t][j] = xs[(xg[t] * 4 + j) * 64];
    };

    float4v acc[RT][NTG];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int t = 0; t < NTG; ++t) acc[r][t] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    float4v acc_a[NTG];  // LA: element v of lane (lr, g) = t[token 16 (tg0 + t) + lr][rank 4 g + v], this wave's K slice
#pragma unroll
    for (int t = 0; t < NTG; ++t) acc_a[t] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

    auto compute = [&](const Unit& u, uint32_t i) {
        const bool live = (wave + i * kWavesK) * 4 + g < nb;  // K tail: a block past the end of the row counts as zero
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            uint32_t sb;
            if constexpr (FMT == 1) sb = live ? static_cast<uint32_t>(u.wb[r].d) : 0u;  // scale only
            else sb = live ? u.wb[r].sb : 0u;
            const half2v d2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x01000100u));
            const half2v b2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x03020302u));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                U4 a;
                if constexpr (FMT == 0) a = dequant8(live ? u.wb[r].q[j] : 0u, d2, b2);
                else if constexpr (FMT == 1) a = dequant8_q8(u.wb[r].q[2 * j], u.wb[r].q[2 * j + 1], d2);
                else a = dequant8_q3(u.wb[r], j, d2, b2);
#pragma unroll
                for (int t = 0; t < NTG; ++t)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, a), __builtin_bit_cast(half8, u.x[t][j]), acc[r][t], 0, 0, 0);
            }
        }
        if constexpr (LA) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int t = 0; t < NTG; ++t)
                    acc_a[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, u.a[j]), __builtin_bit_cast(half8, u.x[t][j]), acc_a[t], 0, 0, 0);
        }
    };

    // Two units in flight.  Every unit that has a successor two places on prefetches it without a
    // condition; the last two or three units are written out.  (A redundant clamped prefetch instead
    // would be waited for by whatever reuses its registers.)
    // (the scheduling fences keep a unit's arithmetic from being hoisted across the loads around it,
    // which would hold both units' temporaries live at once and spill)
#define LQ4_FENCE() __builtin_amdgcn_sched_barrier(0)
    if (cnt > 1) {
        Unit u0, u1;
        load(u0, 0);
        load(u1, 1);
        LQ4_FENCE();
        uint32_t i = 0;
        for (; i + 3 < cnt; i += 2) {
            compute(u0, i);
            LQ4_FENCE();
            load(u0, i + 2);
            LQ4_FENCE();
            compute(u1, i + 1);
            LQ4_FENCE();
            load(u1, i + 3);
            LQ4_FENCE();
        }
        if (cnt - i == 3) {
            compute(u0, i);
            LQ4_FENCE();
            load(u0, i + 2);
            LQ4_FENCE();
            compute(u1, i + 1);
            LQ4_FENCE();
            compute(u0, i + 2);
        } else {
            compute(u0, i);
            LQ4_FENCE();
            compute(u1, i + 1);
        }
    } else if (cnt == 1) {
        Unit u0;
        load(u0, 0);
        compute(u0, 0);
    }
#undef LQ4_FENCE

    // ---- LoRA: wave w adds the ranks w, w + 8, ... of scale * B[row, :] . t[token, :] to its own
    //      partial result in f32, so the delta is spread over all waves and joins the same reduction
    constexpr int kSlot = RT * NTG * 64;
    float* const t_full = reinterpret_cast<float*>(red + 4 * kSlot + kWavesK * NTG * 64);  // [token of the tile][16]
    if constexpr (LA) {
        // the eight K slices of t meet in LDS; every (token, rank) is summed in wave order by one thread
        float4v* const t_part = red + 4 * kSlot;
#pragma unroll
        for (int t = 0; t < NTG; ++t) t_part[(wave * NTG + t) * 64 + lane] = acc_a[t];
        __syncthreads();
        for (uint32_t e = threadIdx.x; e < NTG * 64; e += 64 * kWavesK) {
            float4v sum = t_part[e];
#pragma unroll
            for (int wv = 1; wv < kWavesK; ++wv) sum += t_part[wv * NTG * 64 + e];
            const uint32_t tg = e >> 6, ln = e & 63;  // token 16 tg + ln % 16, ranks 4 (ln / 16) ..
            *reinterpret_cast<float4v*>(t_full + (16 * tg + (ln & 15)) * 16 + 4 * (ln >> 4)) = sum;
        }
        __syncthreads();
    }
    if (lora.rank) {
        auto add_rank = [&](uint32_t jj, const float (&bv)[RT][4]) {
            float tv[NTG];
#pragma unroll
            for (int t = 0; t < NTG; ++t) {
                if constexpr (LA) {
                    tv[t] = t_full[(16 * t + lr) * 16 + jj];
                } else {
                    uint32_t tok = 16 * (tg0 + t) + lr;
                    tok = tok < m ? tok : m - 1;
                    tv[t] = lora.t[static_cast<size_t>(tok) * lora.rank + jj];
                }
            }
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < NTG; ++t)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[r][t][v] = fmaf(bv[r][v], tv[t], acc[r][t][v]);
        };
#pragma unroll
        for (int p = 0; p < 2; ++p) {  // the two ranks whose B was requested at the start
            const uint32_t jj = wave + p * kWavesK;
            if (kEarlyB && jj < lora.rank) {
                float bv[RT][4];
#pragma unroll
                for (int r = 0; r < RT; ++r)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        bv[r][v] = lora.scale * (lora.b_is_f16 ? f16_bits_to_f32(b_raw[p][r][v])
                                                               : __builtin_bit_cast(float, b_raw[p][r][v]));
                add_rank(jj, bv);
            }
        }
        for (uint32_t jj = wave + (kEarlyB ? 2 * kWavesK : 0); jj < lora.rank; jj += kWavesK) {  // the other ranks
            float bv[RT][4];
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    uint32_t row = n0 + 16 * r + 4 * g + v;
                    row = row < n ? row : n - 1;
                    bv[r][v] = lora.scale * load_b(lora.b, lora.b_is_f16, static_cast<size_t>(row) * lora.rank + jj);
                }
            add_rank(jj, bv);
        }
    }

    // ---- the eight K slices meet in LDS in three rounds: (w, w + 4), then (w, w + 2), then (0, 1);
    //      the order is fixed, so the result does not depend on timing
#pragma unroll
    for (int half = kWavesK / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < NTG; ++t) red[(wave - half) * kSlot + (r * NTG + t) * 64 + lane] = acc[r][t];
        }
        __syncthreads();
        if (wave < half) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < NTG; ++t) acc[r][t] += red[wave * kSlot + (r * NTG + t) * 64 + lane];
        }
        if (half > 1) __syncthreads();  // the slots are reused by the next round
    }
    if (wave > 0) return;

    // element v of acc[r][t] in lane (lr, g): token 16 (tg0 + t) + lr, weight row n0 + 16 r + 4 g + v
    const bool vec_ok = (n & 3u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0;
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const uint32_t gn = n0 + 16 * r + 4 * g;
        if (gn >= n) continue;
#pragma unroll
        for (int t = 0; t < NTG; ++t) {
            const uint32_t tok = 16 * (tg0 + t) + lr;
            if (static_cast<uint32_t>(t) >= ntg || tok >= m) continue;
            const float4v val = acc[r][t];
            float* dst = y + static_cast<size_t>(tok) * n + gn;
            if (vec_ok) {
                *reinterpret_cast<float4v*>(dst) = val;
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (gn + v < n) dst[v] = val[v];
            }
        }
    }
}

template <int RT, int FMT, int NTG>
void launch_ntg(const uint8_t* w, uint32_t n, uint32_t k, const uint4* xp, uint32_t m, float* y,
                const LoraEpilogue& lora, hipStream_t stream) {
    const uint32_t groups = (m + 15) / 16;
    const size_t lds = static_cast<size_t>(kWavesK / 2) * RT * NTG * 64 * sizeof(float4v);
    if constexpr (FMT == 0 && RT == 1 && NTG <= 2) {
        if (lora.rank && lora.a) {  // t = A . X inside the launch: the waves' partial t and t itself behind the slots
            const dim3 grid((n + 15) / 16, (groups + NTG - 1) / NTG);
            const size_t lds_t = lds + static_cast<size_t>(kWavesK) * NTG * 64 * sizeof(float4v) + NTG * 16 * 16 * sizeof(float);
            hipLaunchKernelGGL((gemm_q4_skinny<RT, FMT, NTG, true>), grid, dim3(64 * kWavesK), lds_t, stream, w, n, k, xp, m,
                               y, lora, static_cast<uint32_t>(NTG));
            return;
        }
    }
    if (NTG == 2 && groups > 2) {  // tiles of two token groups (launch_rt decides when)
        const dim3 grid2((n + 16 * RT - 1) / (16 * RT), (groups + 1) / 2);
        hipLaunchKernelGGL((gemm_q4_skinny<RT, FMT, NTG>), grid2, dim3(64 * kWavesK), lds, stream, w, n, k, xp, m, y, lora, 2u);
        return;
    }
    const dim3 grid((n + 16 * RT - 1) / (16 * RT), (m + kTokens - 1) / kTokens);
    hipLaunchKernelGGL((gemm_q4_skinny<RT, FMT, NTG>), grid, dim3(64 * kWavesK), lds, stream, w, n, k, xp, m, y, lora,
                       static_cast<uint32_t>(kTokens / 16));
}

// Widest row tile (of 1 or 2) whose two units in flight fit the 256 registers of a wave without spilling.
constexpr int max_rt(int fmt, int ntg) {
    if (fmt == 0) return 2;
    if (fmt == 1) return ntg == 4 ? 1 : 2;
    return ntg == 1 ? 2 : 1;
}

template <int RT, int FMT>
void launch_rt(const uint8_t* w, uint32_t n, uint32_t k, const uint4* xp, uint32_t m, float* y, const LoraEpilogue& lora,
               hipStream_t stream) {
    const uint32_t groups = (m + 15) / 16;
    if (lora.rank && lora.a) {
        // with A as one more tile in the K loop neither a second row tile nor four token groups fit the registers:
        // one row tile, and tiles of two token groups from 33 tokens on (more workgroups, each re-reading its rows)
        if constexpr (RT > 1) return launch_rt<1, FMT>(w, n, k, xp, m, y, lora, stream);
        if (groups > 2) return launch_ntg<1, FMT, 2>(w, n, k, xp, m, y, lora, stream);
    }
    if constexpr (RT == 1 && FMT == 0) {  // (measured for Q4 only)
        // Token tiles of 32 instead of 64 where that fills the chip better: twice the workgroups, each 0.6-0.65 of the
        // time (its rows are read once more, its fixed parts stay).  One workgroup runs per CU, so it pays when the
        // workgroups of the 64-token form are at most half the CUs, or leave the second round of workgroups at most
        // half full (measured at 64 tokens, us: 2048 x 2048 8.15 -> 6.91, 512 x 2048 7.63 -> 6.21, 2048 x 6144 14.9 ->
        // 11.2, 2048 x 12288 30.7 -> 22.9, 5120 x 5120 26.6 -> 23.0, 6144 x 2048 12.8 -> 11.0; against 3072 x 2048 8.23 ->
        // 8.72, 4096 x 2048 8.44 -> 8.80, 4096 x 4096 12.5 -> 13.6, which keep 64).
        const uint32_t wgs = ((n + 15) / 16) * ((m + kTokens - 1) / kTokens);
        if (groups > 2 && (wgs <= 128 || (wgs > 256 && wgs <= 384)))
            return launch_ntg<1, FMT, 2>(w, n, k, xp, m, y, lora, stream);
    }
    if (groups == 1) launch_ntg<(RT < max_rt(FMT, 1) ? RT : max_rt(FMT, 1)), FMT, 1>(w, n, k, xp, m, y, lora, stream);
    else if (groups == 2) launch_ntg<(RT < max_rt(FMT, 2) ? RT : max_rt(FMT, 2)), FMT, 2>(w, n, k, xp, m, y, lora, stream);
    else launch_ntg<(RT < max_rt(FMT, 4) ? RT : max_rt(FMT, 4)), FMT, 4>(w, n, k, xp, m, y, lora, stream);
}

}  // namespace

// The few-token kernel computes t = A . X itself (LoraEpilogue::a set, no launch for t) for Q4, ranks up to 16 and
// up to 64 tokens (q and v of the 2B model, rank 16, 64 tokens: 13.6 us with a launch for t -> 8.3 / 7.7, against
// 8.0 / 7.6 without an adapter).  From 65 tokens on its tiles of 32 tokens are three or four to a row tile: taken
// while those workgroups still find a CU each (512 x 2048 at 128 tokens 10.2 -> 8.0 us; 2048 x 2048, 512 workgroups,
// 12.8 -> 13.0 and left with the launch for t).
bool gemm_skinny_packs_lora_a(uint32_t rank) { return rank != 0 && rank <= 16; }
bool gemm_skinny_computes_t(uint32_t rank, uint32_t m, uint32_t n) {
    if (!gemm_skinny_packs_lora_a(rank)) return false;
    const uint32_t groups = (m + 15) / 16;
    return m <= kTokens || ((n + 15) / 16) * ((groups + 1) / 2) <= 256;
}

// A [rank <= 16, K] (f32 or f16, host memory) as the kernel's matrix-core operand, f16: for K step s (128 wide) and
// instruction j the 64 lanes' 16-byte operands are contiguous; lane (r = lane % 16, g = lane / 16) holds row r,
// K offsets 128 s + 32 g + 8 j .. + 7 in the order x0 x4 x1 x5 x2 x6 x3 x7 of the packed activations.  Rows past
// the rank and K past the end are zero.  (Read row by row, sixteen rows K * 2 bytes apart, every workgroup's loads
// of a step fell on a few memory channels at once and the launch took 4 us longer.)
size_t gemm_skinny_packed_lora_a_bytes(uint32_t k) { return static_cast<size_t>((k + TK - 1) / TK) * 4 * 64 * 16; }
void gemm_skinny_pack_lora_a(const void* a, int a_is_f16, uint32_t rank, uint32_t k, void* out) {
    _Float16* dst = static_cast<_Float16*>(out);
    const uint32_t steps = (k + TK - 1) / TK;
    for (uint32_t s = 0; s < steps; ++s)
        for (uint32_t j = 0; j < 4; ++j)
            for (uint32_t lane = 0; lane < 64; ++lane) {
                const uint32_t r = lane % 16, g = lane / 16;
                const uint32_t k0 = s * TK + 32 * g + 8 * j;
                _Float16* o = dst + ((static_cast<size_t>(s) * 4 + j) * 64 + lane) * 8;
                for (uint32_t e = 0; e < 8; ++e) {
                    const uint32_t src = (e >> 1) + 4 * (e & 1);  // x0 x4 x1 x5 x2 x6 x3 x7
                    float v = 0.0f;
                    if (r < rank && k0 + src < k) {
                        const size_t idx = static_cast<size_t>(r) * k + k0 + src;
                        v = a_is_f16 ? static_cast<float>(static_cast<const _Float16*>(a)[idx]) : static_cast<const float*>(a)[idx];
                    }
                    o[e] = static_cast<_Float16>(v);
                }
            }
}

bool gemm_skinny_wants(uint32_t n, uint32_t k, uint32_t m) {
    // Against the large-tile kernel, which wastes the empty part of its 128-token tile but shares the
    // activations of a tile among 256 rows where this kernel re-reads them for every 16..64 rows
    // (measured on 6M..500M-weight matrices): up to 16 tokens are always served here; one token tile
    // unless the matrix is large
    // (above 2^26 weights) and either more than 32 tokens, fewer than 8192 rows (too few workgroups
    // here) or more than 2^28 weights; two token tiles only up to 2^24 weights.
    if (k < kBlockWeights) return false;
    const uint64_t weights = static_cast<uint64_t>(n) * k;
    if (m <= 16) return true;
    if (m <= kTokens) return weights <= (1ull << 26) || (m <= 32 && n >= 8192 && weights <= (1ull << 28));
    return m <= 2 * kTokens && weights <= (1ull << 24);
}

size_t gemm_skinny_scratch_bytes(uint32_t k, uint32_t m) {
    const size_t steps = (k / kBlockWeights + 3) / 4, groups = (m + 15) / 16;
    return steps * groups * 256 * sizeof(uint4);
}

namespace {

template <int FMT>
void launch_fmt(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                const LoraEpilogue& lora, void* packed_x, hipStream_t stream, bool pack) {
    const uint32_t steps = (k / kBlockWeights + 3) / 4, groups = (m + 15) / 16;
    uint4* xp = static_cast<uint4*>(packed_x);
    constexpr bool kInterleave = FMT == 0;
    if (!pack) {
    } else if (x_is_f16)
        hipLaunchKernelGGL((pack_x_kernel<true, kInterleave>), dim3(steps, groups), dim3(256), 0, stream, x, m, k, xp);
    else
        hipLaunchKernelGGL((pack_x_kernel<false, kInterleave>), dim3(steps, groups), dim3(256), 0, stream, x, m, k, xp);
    // Every workgroup reads the whole packed X of its token tile, so a wider row tile halves that
    // traffic, at the price of fewer workgroups to balance over the compute units.  Measured over
    // 2048..34816 rows and K 2048..17408 at 16, 32 and 64 tokens: two row tiles pay on tall matrices,
    // on long rows and with four token groups; four never do since the K loop keeps two units in flight.
    const uint32_t tiles16 = (n + 15) / 16;
    const bool wide = tiles16 >= 1024 || (k >= 8192 && tiles16 >= 256) || (m > 32 && tiles16 >= 512);
    if (wide) launch_rt<2, FMT>(w, n, k, xp, m, y, lora, stream);
    else launch_rt<1, FMT>(w, n, k, xp, m, y, lora, stream);
}

}  // namespace

void launch_gemm_skinny(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                        const LoraEpilogue& lora, void* packed_x, hipStream_t stream, int fmt, bool pack) {
    if (fmt == 1) launch_fmt<1>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream, pack);
    else if (fmt == 2) launch_fmt<2>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream, pack);
    else launch_fmt<0>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream, pack);
}

}  // namespace lq4
