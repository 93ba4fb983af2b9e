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
// last group and drops the results.  Fixed per instantiation, like the prefetches of the K loop below:
// a load behind a run-time condition makes the compiler wait for loads it cannot count, and the
// pipeline collapses to one unit in flight.
template <int RT, int FMT, int NTG>
__global__ __launch_bounds__(64 * kWavesK) void gemm_q4_skinny(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                                const uint4* __restrict__ xp, uint32_t m,
                                                                float* __restrict__ y, LoraEpilogue lora) {
    extern __shared__ float4v red[];  // 4 slots of RT * 4 * 64 accumulators

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lr = lane & 15;
    const int g = lane >> 4;

    const uint32_t n0 = blockIdx.x * (16 * RT);
    const uint32_t groups = (m + 15) / 16;             // token groups in X (and in the packed image)
    const uint32_t tg0 = blockIdx.y * (kTokens / 16);  // first token group of this workgroup
    const uint32_t ntg = groups - tg0 < 4 ? groups - tg0 : 4;
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

    struct Unit {
        WBlock wb[RT];
        uint4 x[NTG][4];  // [token group][instruction]
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
    if (lora.rank) {
        for (uint32_t jj = wave; jj < lora.rank; jj += kWavesK) {
            float bv[RT][4], tv[NTG];
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    uint32_t row = n0 + 16 * r + 4 * g + v;
                    row = row < n ? row : n - 1;
                    bv[r][v] = lora.scale * load_b(lora.b, lora.b_is_f16, static_cast<size_t>(row) * lora.rank + jj);
                }
#pragma unroll
            for (int t = 0; t < NTG; ++t) {
                uint32_t tok = 16 * (tg0 + t) + lr;
                tok = tok < m ? tok : m - 1;
                tv[t] = lora.t[static_cast<size_t>(tok) * lora.rank + jj];
            }
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < NTG; ++t)
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[r][t][v] = fmaf(bv[r][v], tv[t], acc[r][t][v]);
        }
    }

    // ---- the eight K slices meet in LDS in three rounds: (w, w + 4), then (w, w + 2), then (0, 1);
    //      the order is fixed, so the result does not depend on timing
    constexpr int kSlot = RT * NTG * 64;
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
    const dim3 grid((n + 16 * RT - 1) / (16 * RT), (m + kTokens - 1) / kTokens);
    const size_t lds = static_cast<size_t>(kWavesK / 2) * RT * NTG * 64 * sizeof(float4v);
    hipLaunchKernelGGL((gemm_q4_skinny<RT, FMT, NTG>), grid, dim3(64 * kWavesK), lds, stream, w, n, k, xp, m, y, lora);
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
    if (groups == 1) launch_ntg<(RT < max_rt(FMT, 1) ? RT : max_rt(FMT, 1)), FMT, 1>(w, n, k, xp, m, y, lora, stream);
    else if (groups == 2) launch_ntg<(RT < max_rt(FMT, 2) ? RT : max_rt(FMT, 2)), FMT, 2>(w, n, k, xp, m, y, lora, stream);
    else launch_ntg<(RT < max_rt(FMT, 4) ? RT : max_rt(FMT, 4)), FMT, 4>(w, n, k, xp, m, y, lora, stream);
}

}  // namespace

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
                const LoraEpilogue& lora, void* packed_x, hipStream_t stream) {
    const uint32_t steps = (k / kBlockWeights + 3) / 4, groups = (m + 15) / 16;
    uint4* xp = static_cast<uint4*>(packed_x);
    constexpr bool kInterleave = FMT == 0;
    if (x_is_f16)
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
                        const LoraEpilogue& lora, void* packed_x, hipStream_t stream, int fmt) {
    if (fmt == 1) launch_fmt<1>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream);
    else if (fmt == 2) launch_fmt<2>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream);
    else launch_fmt<0>(w, n, k, x, x_is_f16, m, y, lora, packed_x, stream);
}

}  // namespace lq4
