// Prefill GEMM over native Q4 blocks: Y[M,N] = X[M,K] . W[N,K]^T, f16 operands into the
// matrix cores, f32 accumulate.
//
// Tile: 128 tokens x BN weight rows (128 or 256) x 64 K per step; one wave per 64x64 of
// outputs (2x2 tiles of v_mfma_f32_32x32x16_f16), so 4 or 8 waves per workgroup.  A K step
// consumes two Q4 blocks per weight row: 2*BN blocks per tile, one per thread.  Each thread
// dequantises its block in registers to f16 — "half(f32(q)*d + b)", the rounding point of the
// reference's tiled kernel (shaders/gemm_q4_tiled.metal:57-66) — and stores it beside the f16
// activation tile in LDS.  LDS is double buffered, so a step costs one barrier; activation
// loads run one step ahead of the matrix cores (they mostly hit L2), weight loads three steps
// ahead (they stream from HBM).
//
// With 64 x 64 wave tiles the LDS operand reads alone need the full LDS bandwidth at matrix-core
// peak, so this kernel tops out near a third of peak.  The weights-in-registers kernel
// (lq4_gemm_wreg.hip) serves Q4 and Q3 by default; this one serves Q8_0 on short or narrow
// matrices and stays selectable for the others (block format = template argument FMT).  With
// fewer tiles than workgroup slots it cuts K into ranges, one workgroup per (tile, range), and
// gemm_sum_slices adds the partial tiles in range order.
//
// Dequantisation is done two weights per instruction: a masked dword OR-ed into the mantissa
// of 1024.0 (or 64.0) is the f16 pair (1024+n_lo, 1024+n_hi); one packed subtract makes it
// (n_lo, n_hi) exactly and one packed fma applies scale and bias with a single rounding.
//
// Tiles are numbered so that the workgroups resident at one time, and in particular those
// that share an XCD (consecutive workgroup ids go round-robin over the 8 XCDs), work on a
// small set of token tiles: their activations stay in that XCD's L2 while weights stream.
#include <stdlib.h>

#include <atomic>

#include "lq4_internal.hpp"

namespace lq4 {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int BM = 128;         // tokens per workgroup
constexpr int BK = 64;          // two Q4 blocks along K
constexpr int kPitch = BK + 8;  // halfs per LDS row: 144 bytes keeps 16-byte reads conflict-free
constexpr int kGroupM = 16;     // token tiles per rasterisation group

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

__device__ __forceinline__ float load_b(const void* b, int is_f16, size_t idx) {
    return is_f16 ? static_cast<float>(static_cast<const _Float16*>(b)[idx])
                  : static_cast<const float*>(b)[idx];
}

__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
    return r;
}

__device__ __forceinline__ half2v as_h2(uint32_t v) { return __builtin_bit_cast(half2v, v); }
__device__ __forceinline__ uint32_t as_u32(half2v v) { return __builtin_bit_cast(uint32_t, v); }

// One packed dword (weights 8j..8j+7) -> 8 f16 weights in memory order.
__device__ __forceinline__ uint4 dequant8(uint32_t q, half2v d2, half2v b2) {
    const half2v k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
    const half2v k64 = {static_cast<_Float16>(64.0f), static_cast<_Float16>(64.0f)};
    const uint32_t q8 = q >> 8;
    // pairs (n0,n4) (n1,n5) (n2,n6) (n3,n7)
    const half2v p04 = as_h2(and_or(q, 0x000F000Fu, 0x64006400u)) - k1024;
    const half2v p15 = as_h2(and_or(q, 0x00F000F0u, 0x54005400u)) - k64;
    const half2v p26 = as_h2(and_or(q8, 0x000F000Fu, 0x64006400u)) - k1024;
    const half2v p37 = as_h2(and_or(q8, 0x00F000F0u, 0x54005400u)) - k64;
    const half2v w04 = __builtin_elementwise_fma(p04, d2, b2);
    const half2v w15 = __builtin_elementwise_fma(p15, d2, b2);
    const half2v w26 = __builtin_elementwise_fma(p26, d2, b2);
    const half2v w37 = __builtin_elementwise_fma(p37, d2, b2);
    // back to memory order: (w0,w1) (w2,w3) (w4,w5) (w6,w7)
    uint4 r;
    r.x = __builtin_amdgcn_perm(as_u32(w15), as_u32(w04), 0x05040100u);
    r.y = __builtin_amdgcn_perm(as_u32(w37), as_u32(w26), 0x05040100u);
    r.z = __builtin_amdgcn_perm(as_u32(w15), as_u32(w04), 0x07060302u);
    r.w = __builtin_amdgcn_perm(as_u32(w37), as_u32(w26), 0x07060302u);
    return r;
}

// Q8_0 sibling format (FMT == 1): 34-byte block [u16 f16 scale][32 x i8], only 2-byte aligned.
struct __attribute__((packed, aligned(2))) Q8BlockRaw {
    uint16_t d;
    uint32_t q[8];  // weight i in byte i
};

// Q3 sibling format (FMT == 2): 16-byte block [f16 scale][f16 bias][low-2-bit plane][high-1-bit plane].
struct __attribute__((packed, aligned(4))) Q3BlockRaw {
    uint32_t sb;
    uint32_t lo[2];  // weight i of 16-weight half h at bits 2i of lo[h]
    uint32_t hi;     // weight i at bit i
};

template <int FMT>
struct WBlockOf {
    typedef Q4BlockRaw type;
};
template <>
struct WBlockOf<1> {
    typedef Q8BlockRaw type;
};
template <>
struct WBlockOf<2> {
    typedef Q3BlockRaw type;
};

// Weights 8j..8j+7 of a Q3 block -> 8 f16 weights half(q * d + b) in memory order, q = low2 | hi << 2.
__device__ __forceinline__ uint4 dequant8_q3(const Q3BlockRaw& b, int j, half2v d2, half2v b2) {
    const half2v k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
    const uint32_t lw = (b.lo[j >> 1] >> (16 * (j & 1))) & 0xffffu;  // 8 two-bit fields
    const uint32_t hw = (b.hi >> (8 * j)) & 0xffu;                   // 8 bits
    uint32_t out[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t l4 = lw >> (4 * p), h2 = hw >> (2 * p);
        const uint32_t qa = (l4 & 3u) | ((h2 & 1u) << 2);
        const uint32_t qb = ((l4 >> 2) & 3u) | ((h2 & 2u) << 1);
        const half2v q2 = as_h2(0x64006400u | qa | (qb << 16)) - k1024;
        out[p] = as_u32(__builtin_elementwise_fma(q2, d2, b2));
    }
    return make_uint4(out[0], out[1], out[2], out[3]);
}

// Two packed dwords of a Q8_0 block (weights 8j..8j+7) -> 8 f16 weights half(q * d) in memory
// order.  A sign-flipped byte (q + 128) placed under the exponent byte of 1024.0 is 1024 + 128 + q
// exactly; one packed subtract leaves q, one packed multiply applies the scale with one rounding.
__device__ __forceinline__ uint4 dequant8_q8(uint32_t qa, uint32_t qb, half2v d2) {
    const half2v k1152 = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    const uint32_t ua = qa ^ 0x80808080u, ub = qb ^ 0x80808080u;
    const half2v p01 = as_h2(__builtin_amdgcn_perm(0x64646464u, ua, 0x04010400u)) - k1152;
    const half2v p23 = as_h2(__builtin_amdgcn_perm(0x64646464u, ua, 0x04030402u)) - k1152;
    const half2v p45 = as_h2(__builtin_amdgcn_perm(0x64646464u, ub, 0x04010400u)) - k1152;
    const half2v p67 = as_h2(__builtin_amdgcn_perm(0x64646464u, ub, 0x04030402u)) - k1152;
    uint4 r;
    r.x = as_u32(p01 * d2);
    r.y = as_u32(p23 * d2);
    r.z = as_u32(p45 * d2);
    r.w = as_u32(p67 * d2);
    return r;
}

// BN_: weight rows per workgroup (128 or 256); 2*BN_ threads; waves in a 2 x (BN_/64) grid.
// LORA: compiled with the LoRA step (kept out of the plain kernel, whose register allocation it
// would disturb).
// FMT: 0 = Q4 blocks, 1 = Q8_0 blocks, 2 = Q3 blocks (the siblings have no LoRA step).
//
// K slices.  With fewer tiles than workgroup slots the launch cuts K into `slices.count` ranges of
// `slices.steps` K steps: workgroup b computes tile b / count over range b % count and stores its
// partial tile, row-major [BM][BN_], at slices.partial[b]; gemm_sum_slices adds the ranges of a tile
// in order.  count == 1 writes y directly.
struct KSlices {
    uint32_t count;
    uint32_t steps;
    float* partial;
};

template <bool X_F16, int BN_, bool LORA, int FMT = 0>
__global__ __launch_bounds__(2 * BN_, BN_ == 128 ? 2 : 1) void gemm_q4_mfma(
    const uint8_t* __restrict__ w, uint32_t n, uint32_t k, const void* __restrict__ xv, uint32_t m,
    float* __restrict__ y, LoraEpilogue lora, KSlices slices) {
    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];  // 2 x (X tile | W tile)
    constexpr int kThreads = 2 * BN_;
    constexpr int kWavesN = BN_ / 64;
    constexpr int kTileHalfs = (BM + BN_) * kPitch;
    constexpr int kChunksPerRow = X_F16 ? 8 : 16;       // 16-byte chunks per 64-wide row
    constexpr int XCH = BM * kChunksPerRow / kThreads;  // activation chunks per thread per step

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = (wave / kWavesN) * 64;  // wave's 64x64 sub-tile inside the workgroup tile
    const int wn = (wave % kWavesN) * 64;

    // ---- tile id -> (token tile, weight tile), grouped so co-resident tiles share activations
    const uint32_t tile = blockIdx.x / slices.count;
    const uint32_t slice = blockIdx.x - tile * slices.count;
    const uint32_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN_ - 1) / BN_;
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = tile / per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t group_m = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
    const uint32_t in_group = tile - group * per_group;
    const uint32_t m0 = (first_m + in_group % group_m) * BM;
    const uint32_t n0 = (in_group / group_m) * BN_;

    // This workgroup's K range in steps; blocks at or past `nb` (the end of the range) count as zeros.
    const uint32_t nb_row = k / kBlockWeights;  // blocks per weight row
    const uint32_t s_begin = slice * slices.steps;
    const uint32_t nb = nb_row < 2 * (s_begin + slices.steps) ? nb_row : 2 * (s_begin + slices.steps);
    const uint32_t nsteps = (nb + 1) / 2;

    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- per-thread staging assignments, fixed for the whole K loop ---------------------------
    // weights: thread -> (row tid/2, block tid%2 of the step)
    const uint32_t w_row = n0 + (tid >> 1);
    const bool w_live_row = w_row < n;
    typedef typename WBlockOf<FMT>::type WBlock;
    const uint32_t* w_ptr =
        reinterpret_cast<const uint32_t*>(w) + static_cast<size_t>(w_live_row ? w_row : 0) * (nb_row * 5);
    const uint8_t* w_ptr8 = w + static_cast<size_t>(w_live_row ? w_row : 0) * (nb_row * (FMT == 2 ? 16 : 34));  // FMT != 0
    const int w_half = tid & 1;
    // activations: chunk i of this thread is (row, part) = divmod(tid + kThreads*i, chunks per row)
    const uint8_t* x_ptr[XCH];
    bool x_live[XCH];
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
        const int c = tid + kThreads * i;
        const int row = c / kChunksPerRow, part = c % kChunksPerRow;
        const uint32_t gm = m0 + row;
        x_live[i] = gm < m;
        x_ptr[i] = static_cast<const uint8_t*>(xv) +
                   (static_cast<size_t>(x_live[i] ? gm : 0) * k) * (X_F16 ? 2 : 4) + part * 16;
    }

    struct XStage {
        uint4 x[XCH];
    };

    // Steps past the end of K (the unrolled loop below may run up to three) load nothing.
    auto load_x = [&](XStage& st, uint32_t s) {
        const bool first_ok = 2 * s < nb;       // the step exists at all
        const bool second_ok = 2 * s + 1 < nb;  // the step's second block exists
        const size_t step_bytes = static_cast<size_t>(s) * BK * (X_F16 ? 2 : 4);
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            const int part = (tid + kThreads * i) % kChunksPerRow;
            const bool in_k = part < kChunksPerRow / 2 ? first_ok : second_ok;
            st.x[i] = (x_live[i] && in_k) ? *reinterpret_cast<const uint4*>(x_ptr[i] + step_bytes)
                                          : make_uint4(0, 0, 0, 0);
        }
    };
    auto load_w = [&](WBlock& wst, uint32_t s) {
        uint32_t blk = s * 2 + w_half;
        if (blk >= nb) blk = nb - 1;
        if constexpr (FMT == 0) wst = *reinterpret_cast<const WBlock*>(w_ptr + blk * 5);
        else wst = *reinterpret_cast<const WBlock*>(w_ptr8 + blk * (FMT == 2 ? 16 : 34));
    };

    auto store_tiles = [&](const XStage& st, const WBlock& wst, uint32_t s, _Float16* xs, _Float16* ws) {
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            const int c = tid + kThreads * i;
            const int row = c / kChunksPerRow, part = c % kChunksPerRow;
            if (X_F16) {
                *reinterpret_cast<uint4*>(&xs[row * kPitch + part * 8]) = st.x[i];
            } else {
                half4 h;
                h[0] = static_cast<_Float16>(__builtin_bit_cast(float, st.x[i].x));
                h[1] = static_cast<_Float16>(__builtin_bit_cast(float, st.x[i].y));
                h[2] = static_cast<_Float16>(__builtin_bit_cast(float, st.x[i].z));
                h[3] = static_cast<_Float16>(__builtin_bit_cast(float, st.x[i].w));
                *reinterpret_cast<half4*>(&xs[row * kPitch + part * 4]) = h;
            }
        }
        const bool live = w_live_row && (s * 2 + w_half) < nb;
        _Float16* dst = &ws[(tid >> 1) * kPitch + w_half * 32];
        if constexpr (FMT == 0) {
            const uint32_t sb = live ? wst.sb : 0u;
            const half2v d2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x01000100u));  // (d, d)
            const half2v b2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x03020302u));  // (b, b)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<uint4*>(dst + j * 8) = dequant8(live ? wst.q[j] : 0u, d2, b2);
        } else if constexpr (FMT == 1) {
            const uint32_t db = live ? wst.d : 0u;
            const half2v d2 = as_h2(db | (db << 16));
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<uint4*>(dst + j * 8) = dequant8_q8(wst.q[2 * j], wst.q[2 * j + 1], d2);
        } else {
            const uint32_t sb = live ? wst.sb : 0u;
            const half2v d2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x01000100u));
            const half2v b2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x03020302u));
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<uint4*>(dst + j * 8) = dequant8_q3(wst, j, d2, b2);
        }
    };

    // Matrix-core work of one K step.  Operand layout of v_mfma_f32_32x32x16_f16: lane l supplies
    // row/col (l & 31), k-slice 8*(l >> 5) .. +7 of a 16-deep sub-step.  The operands of sub-step
    // kk+1 are read from LDS while the instructions of sub-step kk execute.
    auto compute = [&](const _Float16* xs, const _Float16* ws) {
        const int r = lane & 31, ksl = (lane >> 5) * 8;
        const _Float16* xa = &xs[(wm + r) * kPitch + ksl];
        const _Float16* wb = &ws[(wn + r) * kPitch + ksl];
        half8 a[2][2], b[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i) a[0][i] = *reinterpret_cast<const half8*>(xa + i * 32 * kPitch);
#pragma unroll
        for (int j = 0; j < 2; ++j) b[0][j] = *reinterpret_cast<const half8*>(wb + j * 32 * kPitch);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk + 1 < BK / 16) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    a[nxt][i] = *reinterpret_cast<const half8*>(xa + i * 32 * kPitch + (kk + 1) * 16);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    b[nxt][j] = *reinterpret_cast<const half8*>(wb + j * 32 * kPitch + (kk + 1) * 16);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[cur][i], b[cur][j], acc[i][j], 0, 0, 0);
        }
    };

    _Float16* xs0 = lds;
    _Float16* ws0 = xs0 + BM * kPitch;
    _Float16* xs1 = lds + kTileHalfs;
    _Float16* ws1 = xs1 + BM * kPitch;

    // The K loop is unrolled by four so that register sets and LDS buffers have fixed roles at every
    // position (nothing is copied): step s uses activation set s%2, weight set s%4, LDS buffer s%2.
    // Steps past the end of K (at most three) run on zeros, which keeps the body branch-free.
    XStage xa, xb;
    WBlock w0, w1, w2, w3;
    load_x(xa, s_begin);
    load_w(w0, s_begin);
    load_w(w1, s_begin + 1);
    load_w(w2, s_begin + 2);
    for (uint32_t s = s_begin; s < nsteps; s += 4) {
        store_tiles(xa, w0, s, xs0, ws0);
        __syncthreads();
        load_x(xb, s + 1);
        load_w(w3, s + 3);
        compute(xs0, ws0);
        store_tiles(xb, w1, s + 1, xs1, ws1);
        __syncthreads();
        load_x(xa, s + 2);
        load_w(w0, s + 4);
        compute(xs1, ws1);
        store_tiles(xa, w2, s + 2, xs0, ws0);
        __syncthreads();
        load_x(xb, s + 3);
        load_w(w1, s + 5);
        compute(xs0, ws0);
        store_tiles(xb, w3, s + 3, xs1, ws1);
        __syncthreads();
        load_x(xa, s + 4);
        load_w(w2, s + 6);
        compute(xs1, ws1);
    }

    // ---- LoRA: extra K steps of depth 16 over the rank on the matrix cores,
    //      acc[token, n] += sum_r (scale * t[token, r]) * B[n, r].
    // Both factors are split hi + lo/2048 into f16 so the delta keeps f32-level accuracy:
    // t.B = thi.Bhi + tlo.(Bhi/2048) + (thi/2048).Blo; the last term vanishes for f16-stored B.
    if (LORA && lora.rank && slice == 0) {
        const int r = lane & 31;
        for (uint32_t r0 = 0; r0 < lora.rank; r0 += 16) {
            const uint32_t rbase = r0 + 8 * (lane >> 5);  // this lane's eight rank indices
            half8 t_hi[2], t_his[2], t_lo[2], b_hi[2], b_his[2], b_lo[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                uint32_t tok = m0 + wm + i * 32 + r;
                tok = tok < m ? tok : m - 1;
                uint32_t row = n0 + wn + i * 32 + r;
                row = row < n ? row : n - 1;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint32_t idx = rbase + e;
                    const bool in = idx < lora.rank;
                    const float tv = in ? lora.scale * lora.t[static_cast<size_t>(tok) * lora.rank + idx] : 0.0f;
                    const float bv = in ? load_b(lora.b, lora.b_is_f16, static_cast<size_t>(row) * lora.rank + idx) : 0.0f;
                    const _Float16 th = static_cast<_Float16>(tv), bh = static_cast<_Float16>(bv);
                    t_hi[i][e] = th;
                    t_his[i][e] = static_cast<_Float16>(tv * (1.0f / 2048.0f));
                    t_lo[i][e] = static_cast<_Float16>((tv - static_cast<float>(th)) * 2048.0f);
                    b_hi[i][e] = bh;
                    b_his[i][e] = static_cast<_Float16>(bv * (1.0f / 2048.0f));
                    b_lo[i][e] = static_cast<_Float16>((bv - static_cast<float>(bh)) * 2048.0f);
                }
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(t_hi[i], b_hi[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(t_lo[i], b_his[j], acc[i][j], 0, 0, 0);
                    if (!lora.b_is_f16)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(t_his[i], b_lo[j], acc[i][j], 0, 0, 0);
                }
        }
    }

    // ---- epilogue: accumulator element v of lane l is
    //      row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
    if (slices.count > 1) {
        float* ptile = slices.partial + static_cast<size_t>(blockIdx.x) * (BM * BN_);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    ptile[(wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3)) * BN_ + wn + j * 32 + (lane & 31)] =
                        acc[i][j][v];
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t gn = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t gm = m0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (gm < m && gn < n) y[static_cast<size_t>(gm) * n + gn] = acc[i][j][v];
            }
        }
}

// y tile = sum over the K slices of its partial tiles, in slice order.  grid (tiles, BM * BN_ / 1024);
// a thread owns four consecutive weight rows of one token.
template <int BN_>
__global__ __launch_bounds__(256) void gemm_sum_slices(const float* __restrict__ partial, uint32_t count, uint32_t m,
                                                       uint32_t n, float* __restrict__ y) {
    const uint32_t tile = blockIdx.x;
    const uint32_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN_ - 1) / BN_;
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = tile / per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t group_m = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
    const uint32_t in_group = tile - group * per_group;
    const uint32_t m0 = (first_m + in_group % group_m) * BM;
    const uint32_t n0 = (in_group / group_m) * BN_;

    const uint32_t local = (blockIdx.y * 256 + threadIdx.x) * 4;
    const uint32_t token = m0 + local / BN_, row = n0 + local % BN_;
    if (token >= m || row >= n) return;
    const float* src = partial + static_cast<size_t>(tile) * count * (BM * BN_) + local;
    float4v v = *reinterpret_cast<const float4v*>(src);
    for (uint32_t sl = 1; sl < count; ++sl) v += *reinterpret_cast<const float4v*>(src + static_cast<size_t>(sl) * (BM * BN_));
    float* dst = y + static_cast<size_t>(token) * n + row;
    if ((n & 3u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0) {
        *reinterpret_cast<float4v*>(dst) = v;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (row + e < n) dst[e] = v[e];
    }
}

// K slicing of a shape for the tile kernel: slice count and steps per slice.  Two workgroups fit a
// compute unit, so up to 512 run at once; a slice keeps at least eight K steps (a multiple of the
// loop's unroll of four), and its partial tile costs a 64 KB write and read.
struct TileSlices {
    uint32_t count, steps;
};
template <int BN_>
TileSlices plan_tile_slices(uint32_t n, uint32_t k, uint32_t m) {
    const uint32_t tiles = ((n + BN_ - 1) / BN_) * ((m + BM - 1) / BM);
    const uint32_t nsteps = (k / kBlockWeights + 1) / 2;
    const uint32_t slots = BN_ == 128 ? 512 : 256;
    uint32_t want = slots / tiles;
    if (want > 16) want = 16;
    if (want < 2 || nsteps < 16) return {1, nsteps};
    uint32_t per = (nsteps + want - 1) / want;
    per = (per + 3) / 4 * 4;
    if (per < 8) per = 8;
    const uint32_t count = (nsteps + per - 1) / per;
    if (count < 2) return {1, nsteps};
    return {count, per};
}

// partial: scratch of tile_scratch_floats() floats, or nullptr to keep K whole.
template <bool X_F16, int BN_, bool LORA, int FMT = 0>
void launch_tile(const uint8_t* w, uint32_t n, uint32_t k, const void* x, uint32_t m, float* y,
                 const LoraEpilogue& lora, hipStream_t stream, float* partial = nullptr) {
    const uint32_t tiles = ((n + BN_ - 1) / BN_) * ((m + BM - 1) / BM);
    TileSlices ts = plan_tile_slices<BN_>(n, k, m);
    if (!partial || (LORA && lora.rank)) ts = TileSlices{1, (k / kBlockWeights + 1) / 2};
    const KSlices slices{ts.count, ts.steps, partial};
    const size_t lds = 2 * (BM + BN_) * kPitch * sizeof(_Float16);
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemm_q4_mfma<X_F16, BN_, LORA, FMT>), 160 * 1024);
    hipLaunchKernelGGL((gemm_q4_mfma<X_F16, BN_, LORA, FMT>), dim3(tiles * ts.count), dim3(2 * BN_), lds, stream, w, n,
                       k, x, m, y, lora, slices);
    if (ts.count > 1)
        hipLaunchKernelGGL((gemm_sum_slices<BN_>), dim3(tiles, BM * BN_ / 1024), dim3(256), 0, stream, partial, ts.count,
                           m, n, y);
}



}  // namespace

// What a context's kernel choice starts from: the environment variable LQ4_GEMM_KERNEL (0..4).
int gemm_kernel_choice_default() {
    const char* e = getenv("LQ4_GEMM_KERNEL");
    const int v = e ? atoi(e) : 0;
    return v >= 0 && v <= 4 ? v : 0;
}

namespace {

// Which kernel serves a shape.
struct GemmPlan {
    bool wreg;
    bool skinny;
    bool w2;  // the weights-in-registers tile at two workgroups per CU (activations packed first)
};

GemmPlan plan_gemm(uint32_t n, uint32_t k, uint32_t m, int x_is_f16, bool with_lora, int forced) {
    if (forced == 3 || (forced == 0 && gemm_skinny_wants(n, k, m))) return {false, true, false};
    if (forced == 1 || !gemm_wreg_supports(n, k, m, x_is_f16)) return {false, false, false};
    if (!with_lora && (forced == 4 || (forced == 0 && gemm_w2_wants(n, k, m)))) return {false, false, true};
    // The weights-in-registers kernel everywhere else: its scheduling cuts a partly filled last round
    // of tiles into K slices, so it no longer needs many tiles to keep the chip busy.
    return {true, false, false};
}

}  // namespace

bool gemm_takes_few_token_kernel(uint32_t n, uint32_t k, uint32_t m, int x_is_f16, int forced) {
    return plan_gemm(n, k, m, x_is_f16, true, forced).skinny;
}

size_t gemm_scratch_floats(uint32_t n, uint32_t k, uint32_t m, int x_is_f16, bool with_lora, int forced) {
    const GemmPlan p = plan_gemm(n, k, m, x_is_f16, with_lora, forced);
    if (p.skinny) return (gemm_skinny_scratch_bytes(k, m) + sizeof(float) - 1) / sizeof(float);
    if (p.w2) return (gemm_w2_scratch_bytes(n, k, m) + sizeof(float) - 1) / sizeof(float);
    return p.wreg ? gemm_wreg_scratch_floats(n, k, m) : 0;
}

void launch_gemm(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m,
                 float* y, const LoraEpilogue& lora, float* scratch, int forced, hipStream_t stream) {
    const GemmPlan p = plan_gemm(n, k, m, x_is_f16, lora.rank != 0, forced);
    if (p.skinny) return launch_gemm_skinny(w, n, k, x, x_is_f16, m, y, lora, scratch, stream);
    if (p.w2) return launch_gemm_w2(w, n, k, x, x_is_f16, m, y, reinterpret_cast<uint8_t*>(scratch), stream);
    if (p.wreg) return launch_gemm_wreg(w, n, k, x, x_is_f16, m, y, lora, scratch, stream);
    if (lora.rank) {
        if (x_is_f16) launch_tile<true, 128, true>(w, n, k, x, m, y, lora, stream);
        else launch_tile<false, 128, true>(w, n, k, x, m, y, lora, stream);
    } else {
        if (x_is_f16) launch_tile<true, 128, false>(w, n, k, x, m, y, lora, stream);
        else launch_tile<false, 128, false>(w, n, k, x, m, y, lora, stream);
    }
}

// Sibling formats: the weights-in-registers kernel with the format's decoder, unless the tile
// kernel is forced (choice 1).  Q8_0 blocks are 1.7 x the bytes and 2-byte aligned, which costs the
// register kernel more than the tile kernel (measured): it is taken on long, wide matrices only.
namespace {
bool sibling_wants_wreg(int fmt, uint32_t n, uint32_t k, int forced) {
    if (forced == 1) return false;
    if (forced == 2) return true;
    return fmt != 1 || (k >= 4096 && n >= 4096);
}

template <int FMT>
void launch_sibling(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    float* scratch, int forced, hipStream_t stream) {
    const LoraEpilogue none{nullptr, nullptr, 0, 0, 0.0f};
    if (sibling_wants_wreg(FMT, n, k, forced)) return launch_gemm_wreg(w, n, k, x, x_is_f16, m, y, none, scratch, stream, FMT);
    if (x_is_f16) launch_tile<true, 128, false, FMT>(w, n, k, x, m, y, none, stream, scratch);
    else launch_tile<false, 128, false, FMT>(w, n, k, x, m, y, none, stream, scratch);
}
}  // namespace

size_t gemm_sibling_scratch_floats(int fmt, uint32_t n, uint32_t k, uint32_t m, int forced) {
    if (sibling_wants_wreg(fmt, n, k, forced)) return gemm_wreg_scratch_floats(n, k, m);
    const TileSlices ts = plan_tile_slices<128>(n, k, m);
    if (ts.count < 2) return 0;
    return static_cast<size_t>((n + 127) / 128) * ((m + BM - 1) / BM) * ts.count * (BM * 128);
}

void launch_gemm_q8(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    float* scratch, int forced, hipStream_t stream) {
    launch_sibling<1>(w, n, k, x, x_is_f16, m, y, scratch, forced, stream);
}

void launch_gemm_q3(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    float* scratch, int forced, hipStream_t stream) {
    launch_sibling<2>(w, n, k, x, x_is_f16, m, y, scratch, forced, stream);
}

}  // namespace lq4
