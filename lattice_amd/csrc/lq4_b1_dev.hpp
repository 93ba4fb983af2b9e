// Device helpers shared by the batch-1 GEMV kernel, the decode-chain kernel and the per-pair MoE kernels: how a
// lane reads a 20-byte block, how activations are staged in LDS, and the per-block dot product.
//
// Arithmetic.  A naive unpack (shift, mask, int->float, fma per nibble) would make vector issue, not HBM, the
// limit on this chip, and so does any form that touches the nibbles one or two at a time.  Here a packed dword
// is never unpacked: v_dot8_u32_u4 multiplies the eight nibbles of a weight dword with eight 4-bit digits of
// the activations and adds the products, exactly, in one full-rate instruction.
//
// Activations keep f32 accuracy and f32 range: the 32 activations of a block are scaled by the power of two
// above the block's largest magnitude and rounded to 23-bit fixed point, t = rint(x * 2^22 / S), |t| <= 2^22
// (an absolute error of 2^-23 S per activation: the accuracy of an f32 at the block's largest magnitude), and
// x' = t + 2^22 >= 0 is cut into six 4-bit digits.  With A_p = sum_k n_k digit_p(x'_k) (four dot8 per digit)
// and Q = sum_k n_k (four more),
//   sum_k n_k t_k = sum_p 16^p A_p - 2^22 Q,
// an integer below 2^31 computed without rounding, then converted once.  Per block
//   y += d * (S 2^-22) * sum_k n_k t_k  +  b * sum_k x_k,
// the bias-factored form of the reference kernel (shaders/qwen35.metal:838-847), whose one-token kernel reads
// f32 activations (shaders/qwen35.metal:800-847).  28 dot instructions per block and lane, against 20 masks and
// 32 two-wide dot products for the f16 hi/lo form this replaces.
#pragma once

#include "lq4_internal.hpp"

namespace lq4 {
namespace b1 {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Pointers with their address space spelled out.  A pointer the compiler cannot trace back to LDS or
// to a kernel argument becomes a flat access, which counts on both memory counters: every LDS read
// would then wait for the weight loads in flight, and every weight load for the LDS.
#define LQ4_LDS __attribute__((address_space(3)))
#define LQ4_GLOBAL __attribute__((address_space(1)))
typedef LQ4_LDS uint32_t lds_u32;

template <typename T>
__device__ __forceinline__ const LQ4_GLOBAL T* as_global(const T* p) {
    return (const LQ4_GLOBAL T*)p;
}
template <typename T>
__device__ __forceinline__ LQ4_GLOBAL T* as_global(T* p) {
    return (LQ4_GLOBAL T*)p;
}

constexpr int kXPitch = 36;  // dwords of LDS per block of x: 24 digit dwords (dword-column j of digit p at 6j + p),
                             // 8 unused, sum, S * 2^-22, 2 pad (36 keeps 16-byte lane reads at stride 144 B
                             // conflict-free)
constexpr int kDigits = 6;
constexpr float kRoundMagic = 12582912.0f;        // 1.5 * 2^23: x + magic has rint(x) + 2^22 in its low bits
constexpr uint32_t kRoundMagicBits = 0x4B000000u;  // bits of 2^23

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

__device__ __forceinline__ uint32_t udot8(uint32_t a, uint32_t b, uint32_t c) {
    return __builtin_amdgcn_udot8(a, b, c, false);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}

// max with the value of another lane of the quad; v must not be negative
template <int CTRL>
__device__ __forceinline__ float dpp_max_quad(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
    return fmaxf(v, __builtin_bit_cast(float, moved));
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load
// the wave has in flight, i.e. for the weights it requested ahead; LDS writes need no more than
// their own counter before the barrier.
__device__ __forceinline__ void barrier_lds() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Sums groups of SEG adjacent lanes (SEG = 16, 32 or 64); the total of a group is valid
// in its last lane.
template <int SEG>
__device__ __forceinline__ float segment_sum(float v) {
    v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane holds its 16-lane row sum
    if (SEG >= 32) v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    if (SEG >= 64) v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

// Bytes b of four fixed-point values, one per byte: pair() interleaves the low two bytes of two values
// ([a.B0, b.B0, a.B1, b.B1]) or takes their third byte ([a.B2, b.B2, 0, 0]); quad() joins two such pairs.
__device__ __forceinline__ uint32_t perm(uint32_t high, uint32_t low, uint32_t sel) {
    return __builtin_amdgcn_perm(high, low, sel);
}

// Cuts 8 consecutive fixed-point activations x'[i] (24 bits each, the partners of one packed dword: nibble i of
// the dword is weight i) into the six digit dwords: nibble i of out[p] = digit p of x'[i].
__device__ __forceinline__ void digits_x8(const uint32_t (&xf)[8], uint32_t (&out)[kDigits]) {
    uint32_t byte_plane[2][3];  // [even / odd elements][byte]: the bytes of elements (0,2,4,6) or (1,3,5,7)
#pragma unroll
    for (int o = 0; o < 2; ++o) {
        const uint32_t u0 = perm(xf[2 + o], xf[0 + o], 0x05010400u), u1 = perm(xf[6 + o], xf[4 + o], 0x05010400u);
        const uint32_t v0 = perm(xf[2 + o], xf[0 + o], 0x0c0c0602u), v1 = perm(xf[6 + o], xf[4 + o], 0x0c0c0602u);
        byte_plane[o][0] = perm(u1, u0, 0x05040100u);
        byte_plane[o][1] = perm(u1, u0, 0x07060302u);
        byte_plane[o][2] = perm(v1, v0, 0x05040100u);
    }
    constexpr uint32_t kLow = 0x0F0F0F0Fu;
#pragma unroll
    for (int b = 0; b < 3; ++b) {
        const uint32_t ev = byte_plane[0][b], od = byte_plane[1][b];
        out[2 * b] = (ev & kLow) | ((od << 4) & ~kLow);
        out[2 * b + 1] = ((ev >> 4) & kLow) | (od & ~kLow);
    }
}

// Stages unit g = (block g >> 2, dword g & 3) of the activation vector: 8 activations in a, b.  The
// four threads of a block must be four adjacent lanes of one quad, all of them calling together
// (`store` = false for the clamped duplicates past the end of the vector).
__device__ __forceinline__ void stage_x8(lds_u32* xs, uint32_t g, const float4 a, const float4 b, bool store) {
    const uint32_t blk = g >> 2, j = g & 3;
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float sx = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    float m = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                    fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
    // the 4 threads of a block are 4 adjacent lanes: quad butterflies
    sx = dpp_add<0xB1, 0xF>(sx);
    sx = dpp_add<0x4E, 0xF>(sx);
    m = dpp_max_quad<0xB1>(m);
    m = dpp_max_quad<0x4E>(m);
    // S = 2^(e - 126), the power of two above the block's largest magnitude (e its biased exponent; blocks below
    // 2^-103 share that scale, so S * 2^-22 stays a normal number).  to_fixed = 2^22 / S and S * 2^-22 are exact.
    uint32_t e = __builtin_bit_cast(uint32_t, m) >> 23;
    e = e < 23u ? 23u : e > 254u ? 254u : e;
    const float to_fixed = __builtin_bit_cast(float, (275u - e) << 23);
    float scale = __builtin_bit_cast(float, (e - 21u) << 23);
    // an infinite or NaN activation (or a sum that overflows) reaches every row, as it does in f32 arithmetic
    if (!(fabsf(sx) <= 3.402823466e38f)) scale = __builtin_nanf("");
    uint32_t xf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)  // rint(v * to_fixed) + 2^22, rounded to nearest even by the addition itself
        xf[i] = __builtin_bit_cast(uint32_t, fmaf(v[i], to_fixed, kRoundMagic)) - kRoundMagicBits;
    uint32_t dg[kDigits];
    digits_x8(xf, dg);
    if (store) {
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        LQ4_LDS u32x2* dst = reinterpret_cast<LQ4_LDS u32x2*>(&xs[blk * kXPitch + kDigits * j]);
        dst[0] = u32x2{dg[0], dg[1]};
        dst[1] = u32x2{dg[2], dg[3]};
        dst[2] = u32x2{dg[4], dg[5]};
        if (j == 0) *reinterpret_cast<LQ4_LDS f32x2*>(&xs[blk * kXPitch + 32]) = f32x2{sx, scale};
    }
}

// The staged activations of one block, in a lane's registers.
struct XBlock {
    uint32_t n[4 * kDigits];  // digit p of dword-column j at kDigits * j + p
    float sum, scale;         // sum of the block's activations; S * 2^-22
};

__device__ __forceinline__ void load_xblock(const lds_u32* xs, uint32_t blk, XBlock& x) {
    const LQ4_LDS u32x4* xsrc = reinterpret_cast<const LQ4_LDS u32x4*>(&xs[blk * kXPitch]);
#pragma unroll
    for (int i = 0; i < kDigits; ++i) {
        const u32x4 d = xsrc[i];
        x.n[4 * i + 0] = d.x; x.n[4 * i + 1] = d.y; x.n[4 * i + 2] = d.z; x.n[4 * i + 3] = d.w;
    }
    const f32x2 ss = *reinterpret_cast<const LQ4_LDS f32x2*>(&xs[blk * kXPitch + 32]);
    x.sum = ss.x;
    x.scale = ss.y;
}

// sum_k n_k * t_k over one block, t the block's fixed-point activations (exact).
__device__ __forceinline__ float block_dot(const uint32_t (&q)[4], const uint32_t (&xn)[4 * kDigits]) {
    uint32_t part[kDigits], nib = 0;
#pragma unroll
    for (int p = 0; p < kDigits; ++p) part[p] = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int p = 0; p < kDigits; ++p) part[p] = udot8(q[j], xn[kDigits * j + p], part[p]);
        nib = udot8(q[j], 0x11111111u, nib);
    }
    // sum_p 16^p part[p] <= 480 * 2^23 < 2^32; minus 2^22 * nib it is below 2^31 in magnitude
    const uint32_t lo = part[0] + (part[1] << 4) + (part[2] << 8);
    const uint32_t hi = part[3] + (part[4] << 4) + (part[5] << 8);
    const uint32_t total = lo + (hi << 12) - (nib << 22);
    return static_cast<float>(static_cast<int32_t>(total));
}

// acc + (one block of one weight row) . (the staged block x); `live` = false drops the block
// (a lane past the end of the row that re-read a valid block).
__device__ __forceinline__ float block_fma(const Q4BlockRaw& w, const XBlock& x, bool live, float acc) {
    const float p = block_dot(w.q, x.n);
    float d = f16_bits_to_f32(w.sb & 0xffffu);
    const float b = f16_bits_to_f32(w.sb >> 16);
    if (!live) d = 0.0f;
    return fmaf(d * p, x.scale, fmaf(b, live ? x.sum : 0.0f, acc));
}

}  // namespace b1
}  // namespace lq4
