// Device helpers shared by the batch-1 GEMV kernel and the decode-chain kernel: how a lane reads a
// 20-byte block, how activations are staged in LDS, and the per-block dot product.
//
// Arithmetic.  A naive unpack (shift, mask, int->float, fma per nibble) would make vector issue,
// not HBM, the limit on this chip.  Instead a masked dword IS a pair of f16 subnormals:
// q & 0x000F000F = (n_lo, n_hi) * 2^-24 and q & 0x00F000F0 = (n_lo, n_hi) * 2^-20 (gfx950's
// v_dot2_f32_f16 honours f16 subnormals), so one v_and per two weights unpacks them exactly, and
// v_dot2_f32_f16 does two MACs per op with f32 accumulation.  The activations paired with the
// 2^-20 form are pre-scaled by 2^-4.
//
// Activations keep f32 accuracy and f32 range: the 32 activations of a block are divided by
// 2^e, the power of two of the block's largest magnitude, and each quotient is split x = hi + lo/2048
// with hi, lo both f16.  Every product is exact, the result tracks an f32 GEMV (not an f16 one), and
// any finite f32 activation is representable (the reference's one-token kernel reads f32 x,
// shaders/qwen35.metal:800-847).  Per block
//   y += 2^e * (d * 2^24) * sum_k (n_k 2^-24) (x_k / 2^e)  +  b * sum_k x_k,
// the bias-factored form of the reference kernel (shaders/qwen35.metal:838-847).
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

constexpr int kXPitch = 36;  // dwords of LDS per block of x: 16 hi pairs, 16 lo pairs, sum, 2^e, 2 pad
                             // (36 keeps 16-byte lane reads at stride 144 B conflict-free)
constexpr float kLoScale = 2048.0f;
constexpr float kTwo24 = 16777216.0f;

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b), c, false);
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

__device__ __forceinline__ uint32_t pack_h2(_Float16 a, _Float16 b) {
    const half2v h = {a, b};
    return __builtin_bit_cast(uint32_t, h);
}

// Converts 8 consecutive activations (the partners of one packed dword), already divided by the
// block's power of two, into the pair order the unpack produces — (0,4) (1,5) (2,6) (3,7) — as f16 hi
// parts and scaled f16 residuals.  Odd elements pair with the 2^-20 nibble form and are split
// after scaling by 2^-4.
__device__ __forceinline__ void convert_x8(const float (&v)[8], uint4& ph, uint4& pl) {
    _Float16 hi[8], lo[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float s = (i & 1) ? v[i] * 0.0625f : v[i];
        hi[i] = static_cast<_Float16>(s);
        lo[i] = static_cast<_Float16>((s - static_cast<float>(hi[i])) * kLoScale);
    }
    ph.x = pack_h2(hi[0], hi[4]); ph.y = pack_h2(hi[1], hi[5]);
    ph.z = pack_h2(hi[2], hi[6]); ph.w = pack_h2(hi[3], hi[7]);
    pl.x = pack_h2(lo[0], lo[4]); pl.y = pack_h2(lo[1], lo[5]);
    pl.z = pack_h2(lo[2], lo[6]); pl.w = pack_h2(lo[3], lo[7]);
}

// Stages unit g = (block g >> 2, dword g & 3) of the activation vector: 8 activations in a, b.  The
// four threads of a block must be four adjacent lanes of one quad, all of them calling together
// (`store` = false for the clamped duplicates past the end of the vector).
__device__ __forceinline__ void stage_x8(lds_u32* xs, uint32_t g, const float4 a, const float4 b, bool store) {
    const uint32_t blk = g >> 2, j = g & 3;
    float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    float sx = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    float m = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                    fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
    // the 4 threads of a block are 4 adjacent lanes: quad butterflies
    sx = dpp_add<0xB1, 0xF>(sx);
    sx = dpp_add<0x4E, 0xF>(sx);
    m = dpp_max_quad<0xB1>(m);
    m = dpp_max_quad<0x4E>(m);
    // 2^e = the power of two at or below the block's largest magnitude (1 for an all-zero or
    // subnormal block); its reciprocal is exact
    uint32_t e = __builtin_bit_cast(uint32_t, m) >> 23;
    e = e == 0 ? 127u : e > 253u ? 253u : e;
    const float scale = __builtin_bit_cast(float, e << 23);
    const float inv = __builtin_bit_cast(float, (254u - e) << 23);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] *= inv;
    uint4 ph, pl;
    convert_x8(v, ph, pl);
    if (store) {
        *reinterpret_cast<LQ4_LDS u32x4*>(&xs[blk * kXPitch + 4 * j]) = u32x4{ph.x, ph.y, ph.z, ph.w};
        *reinterpret_cast<LQ4_LDS u32x4*>(&xs[blk * kXPitch + 16 + 4 * j]) = u32x4{pl.x, pl.y, pl.z, pl.w};
        if (j == 0) *reinterpret_cast<LQ4_LDS f32x2*>(&xs[blk * kXPitch + 32]) = f32x2{sx, scale};
    }
}

// The staged activations of one block, in a lane's registers.
struct XBlock {
    uint32_t h[16], l[16];
    float sum, scale;
};

__device__ __forceinline__ void load_xblock(const lds_u32* xs, uint32_t blk, XBlock& x) {
    const LQ4_LDS u32x4* xsrc = reinterpret_cast<const LQ4_LDS u32x4*>(&xs[blk * kXPitch]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4 h = xsrc[i], l = xsrc[4 + i];
        x.h[4 * i + 0] = h.x; x.h[4 * i + 1] = h.y; x.h[4 * i + 2] = h.z; x.h[4 * i + 3] = h.w;
        x.l[4 * i + 0] = l.x; x.l[4 * i + 1] = l.y; x.l[4 * i + 2] = l.z; x.l[4 * i + 3] = l.w;
    }
    const f32x2 ss = *reinterpret_cast<const LQ4_LDS f32x2*>(&xs[blk * kXPitch + 32]);
    x.sum = ss.x;
    x.scale = ss.y;
}

// 2^-24 * sum_k n_k * x_k over one block (x as staged: divided by the block's power of two).
__device__ __forceinline__ float block_dot(const uint32_t (&q)[4], const uint32_t (&xh)[16],
                                           const uint32_t (&xl)[16]) {
    float ph = 0.0f, pl = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t w0 = q[j] & 0x000F000Fu;
        const uint32_t w1 = q[j] & 0x00F000F0u;
        const uint32_t q8 = q[j] >> 8;
        const uint32_t w2 = q8 & 0x000F000Fu;
        const uint32_t w3 = q8 & 0x00F000F0u;
        ph = dot2(w0, xh[4 * j + 0], ph);
        pl = dot2(w0, xl[4 * j + 0], pl);
        ph = dot2(w1, xh[4 * j + 1], ph);
        pl = dot2(w1, xl[4 * j + 1], pl);
        ph = dot2(w2, xh[4 * j + 2], ph);
        pl = dot2(w2, xl[4 * j + 2], pl);
        ph = dot2(w3, xh[4 * j + 3], ph);
        pl = dot2(w3, xl[4 * j + 3], pl);
    }
    return fmaf(pl, 1.0f / kLoScale, ph);
}

// acc + (one block of one weight row) . (the staged block x); `live` = false drops the block
// (a lane past the end of the row that re-read a valid block).
__device__ __forceinline__ float block_fma(const Q4BlockRaw& w, const XBlock& x, bool live, float acc) {
    const float p = block_dot(w.q, x.h, x.l);
    float d = f16_bits_to_f32(w.sb & 0xffffu) * kTwo24;
    const float b = f16_bits_to_f32(w.sb >> 16);
    if (!live) d = 0.0f;
    return fmaf(d * p, x.scale, fmaf(b, live ? x.sum : 0.0f, acc));
}

}  // namespace b1
}  // namespace lq4
