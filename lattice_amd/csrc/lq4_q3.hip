// Q3 sibling of the batch-1 decode GEMV:  y[n] = sum_k W[n,k] * x[k]  over 16-byte blocks
// [u16 f16 scale][u16 f16 bias][8 bytes low-2-bit plane][4 bytes high-1-bit plane],
// w = q * scale + bias, q = low2 | hi << 2  (weights/q3_weights.rs:13-52; reference arithmetic
// gemv_q3_reference, weights/q3_weights.rs:784-797: dequantise, then an f32 dot product).
//
// Work layout as in the Q4 kernel: lane l owns block 64 s + l of every row of its wave's chunk
// (1024 contiguous bytes per row and slab), activations staged once per workgroup in LDS.
//
// Arithmetic.  The planes are never unpacked.  A masked plane dword IS a pair of f16 subnormals:
// the low plane keeps weight e of a 16-weight half at bits 2e, so L & (3 << 2e) in both halves
// is (q2[e], q2[e+8]) * 4^e * 2^-24; the high plane keeps weight e at bit e, so H & (1 << e) is
// (hi[e], hi[e+16]) * 2^e * 2^-24.  Only the ten mantissa bits of an f16 can be used that way:
// fields above bit 9 are reached through one shift right by 6.  The activations are staged as
// f16 pairs in the matching order, pre-divided by the field's power of two (and times 4 for the
// high plane), so v_dot2_f32_f16 accumulates 2^-24 * sum q x directly: 17 operations per 16
// low-plane weights, 33 per 32 high-plane bits.  Per block
//   y += (scale * 2^24) * dot + bias * sum_k x_k.
// Activations are rounded to f16 here (relative error of y about 3e-4, far below the format's
// own quantisation step); they must be finite and inside the f16 range.
#include "lq4_internal.hpp"

#include <type_traits>

namespace lq4 {

namespace {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

constexpr int kWaves = 4;
constexpr int kXPitch = 36;  // dwords of LDS per block of x: 8 + 8 low-plane pairs, 16 high-plane pairs, sum, pad
constexpr int kQ3BlockBytes = 16;
constexpr float kTwo24 = 16777216.0f;

struct __attribute__((packed, aligned(4))) Q3BlockRaw {
    uint32_t sb;     // f16 scale | f16 bias << 16
    uint32_t lo[2];  // low-2-bit plane: weight i of half h at bits 2i of lo[h] (16 weights per dword)
    uint32_t hi;     // high-1-bit plane: weight i at bit i
};

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b), c, false);
}

template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over the 64 lanes of a wave with data-parallel-primitive moves only; valid in lane 63.
__device__ __forceinline__ float wave_total(float v) {
    v = dpp_add<0xB1>(v);        // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);        // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);       // row_half_mirror
    v = dpp_add<0x140>(v);       // row_mirror: every lane holds its 16-lane row sum
    v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const half2v h = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
    return __builtin_bit_cast(uint32_t, h);
}

// 2^-24 * sum_i q_i * x_i over one block; xr = the block's 32 staged activation pairs.
__device__ __forceinline__ float block_dot(const Q3BlockRaw& b, const uint32_t (&xr)[32]) {
    float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const uint32_t l = b.lo[h], t = l >> 6;
        s0 = dot2(l & 0x00030003u, xr[8 * h + 0], s0);
        s1 = dot2(l & 0x000C000Cu, xr[8 * h + 1], s1);
        s0 = dot2(l & 0x00300030u, xr[8 * h + 2], s0);
        s1 = dot2(l & 0x00C000C0u, xr[8 * h + 3], s1);
        s0 = dot2(l & 0x03000300u, xr[8 * h + 4], s0);
        s1 = dot2(t & 0x00300030u, xr[8 * h + 5], s1);
        s0 = dot2(t & 0x00C000C0u, xr[8 * h + 6], s0);
        s1 = dot2(t & 0x03000300u, xr[8 * h + 7], s1);
    }
    const uint32_t hb = b.hi, th = hb >> 6;
#pragma unroll
    for (int e = 0; e < 10; e += 2) {
        s0 = dot2(hb & (0x00010001u << e), xr[16 + e], s0);
        s1 = dot2(hb & (0x00010001u << (e + 1)), xr[17 + e], s1);
    }
#pragma unroll
    for (int e = 10; e < 16; e += 2) {
        s0 = dot2(th & (0x00010001u << (e - 6)), xr[16 + e], s0);
        s1 = dot2(th & (0x00010001u << (e - 5)), xr[17 + e], s1);
    }
    return s0 + s1;
}

// Chunk c of wave `wid` holds rows (c * RW + j) * n_waves + wid, j < RW; a unit is one
// (chunk, slab of 64 blocks).  Dynamic LDS: (K/32) * kXPitch dwords.
// HX: 8-activation units per thread requested ahead of the weights (all of K up to 2048 * HX).
template <int RW, int HX>
__global__ __launch_bounds__(kWaves * 64) void gemv_q3_b1(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                          const float* __restrict__ x, float* __restrict__ y) {
    extern __shared__ __attribute__((aligned(16))) uint32_t xs[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t nb = k / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ3BlockBytes;
    const uint32_t slabs = (nb + 63) / 64;
    const uint32_t n_waves = gridDim.x * kWaves;
    const uint32_t wid = __builtin_amdgcn_readfirstlane(blockIdx.x * kWaves + (tid >> 6));
    const uint32_t first = wid < n ? n - wid : 0;
    const uint32_t chunks = (first + n_waves * RW - 1) / (n_waves * RW);
    const uint32_t units = chunks * slabs;

    auto load_unit = [&](Q3BlockRaw (&buf)[RW], uint32_t u) {
        const uint32_t chunk = u / slabs, slab = u - chunk * slabs;
        uint32_t blk = slab * 64 + lane;
        if (blk >= nb) blk = nb - 1;
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            uint32_t row = (chunk * RW + j) * n_waves + wid;
            if (row >= n) row = n - 1;
            buf[j] = *reinterpret_cast<const Q3BlockRaw*>(w + row * row_bytes + blk * static_cast<uint32_t>(kQ3BlockBytes));
        }
    };

    // ---- stage x: four threads per block ------------------------------------------------------
    // thread j = 0, 1: low-plane pairs of weights 16 j .. 16 j + 15; j = 2, 3: high-plane pairs
    // e = 8 (j - 2) .. + 7, i.e. (x[e], x[e + 16]).
    auto x_src = [&](uint32_t g, const float4*& pa, const float4*& pb) {
        const uint32_t blk = g >> 2, j = g & 3;
        const float* xb = x + blk * kBlockWeights;
        pa = reinterpret_cast<const float4*>(xb + (j < 2 ? 16 * j : 8 * (j - 2)));
        pb = reinterpret_cast<const float4*>(xb + (j < 2 ? 16 * j + 8 : 8 * (j - 2) + 16));
    };
    auto stage = [&](uint32_t g, const float4 a0, const float4 a1, const float4 b0, const float4 b1, bool store) {
        const uint32_t blk = g >> 2, j = g & 3;
        const float va[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        const float vb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
        uint32_t out[8];
        float sx = 0.0f;
        if (j < 2) {
            // field e sits at bits 2e (e <= 4) or, after the shift by 6, at bits 2(e - 3)
            const float sc[8] = {1.0f, 0.25f, 0.0625f, 0.015625f, 0.00390625f, 0.0625f, 0.015625f, 0.00390625f};
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = pack_h2(va[e] * sc[e], vb[e] * sc[e]);
            sx = (((va[0] + va[1]) + (va[2] + va[3])) + ((va[4] + va[5]) + (va[6] + va[7]))) +
                 (((vb[0] + vb[1]) + (vb[2] + vb[3])) + ((vb[4] + vb[5]) + (vb[6] + vb[7])));
        } else {
            // bit e of the plane is worth 2^e (e <= 9) or, after the shift by 6, 2^(e - 6); a set bit adds 4 to q
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ee = 8 * (static_cast<int>(j) - 2) + e;
                const int p = ee <= 9 ? ee : ee - 6;
                const float sc = 4.0f / static_cast<float>(1 << p);
                out[e] = pack_h2(va[e] * sc, vb[e] * sc);
            }
        }
        sx = dpp_add<0xB1>(sx);  // the 4 threads of a block are 4 adjacent lanes: quad butterfly
        sx = dpp_add<0x4E>(sx);
        if (store) {
            uint4* dst = reinterpret_cast<uint4*>(&xs[blk * kXPitch + 8 * j]);
            dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
            dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
            if (j == 0) *reinterpret_cast<float*>(&xs[blk * kXPitch + 32]) = sx;
        }
    };

    // The first activations of every thread are requested before any weight (clamped addresses, no
    // branch): loads return in order, so behind the weight prefetch their staging, and the barrier
    // after it, would wait until the first weights have crossed from HBM.
    uint32_t gx[HX];
    float4 xa0[HX], xa1[HX], xb0[HX], xb1[HX];
#pragma unroll
    for (int i = 0; i < HX; ++i) {
        const uint32_t g = tid + i * kWaves * 64;
        gx[i] = g < nb * 4 ? g : 0;
        const float4 *pa, *pb;
        x_src(gx[i], pa, pb);
        xa0[i] = pa[0]; xa1[i] = pa[1]; xb0[i] = pb[0]; xb1[i] = pb[1];
    }

    Q3BlockRaw buf_a[RW], buf_b[RW];
    load_unit(buf_a, 0);  // (a wave without rows re-reads the last row; it stores nothing)
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads

#pragma unroll
    for (int i = 0; i < HX; ++i) stage(gx[i], xa0[i], xa1[i], xb0[i], xb1[i], tid + i * kWaves * 64 < nb * 4);
    for (uint32_t g = tid + HX * kWaves * 64; g < nb * 4; g += kWaves * 64) {
        const float4 *pa, *pb;
        x_src(g, pa, pb);
        stage(g, pa[0], pa[1], pb[0], pb[1], true);
    }
    __syncthreads();

    float acc[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) acc[j] = 0.0f;

    // `prefetch` is a compile-time flag: behind a run-time condition the compiler would have to wait
    // for most of the just-issued next unit before it may use the current one.
    auto process = [&](auto prefetch, Q3BlockRaw (&cur)[RW], Q3BlockRaw (&nxt)[RW], uint32_t u) {
        const uint32_t chunk = u / slabs, slab = u - chunk * slabs;
        if constexpr (decltype(prefetch)::value) load_unit(nxt, u + 1);
        const uint32_t blk_raw = slab * 64 + lane;
        const bool live = blk_raw < nb;
        const uint32_t blk = live ? blk_raw : nb - 1;
        uint32_t xr[32];
        const uint4* xsrc = reinterpret_cast<const uint4*>(&xs[blk * kXPitch]);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint4 v = xsrc[i];
            xr[4 * i + 0] = v.x; xr[4 * i + 1] = v.y; xr[4 * i + 2] = v.z; xr[4 * i + 3] = v.w;
        }
        const float sum_x = live ? *reinterpret_cast<const float*>(&xs[blk * kXPitch + 32]) : 0.0f;
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const float p = block_dot(cur[j], xr);
            float d = f16_bits_to_f32(cur[j].sb & 0xffffu) * kTwo24;
            const float b = f16_bits_to_f32(cur[j].sb >> 16);
            if (!live) d = 0.0f;
            acc[j] = fmaf(d, p, fmaf(b, sum_x, acc[j]));
        }
        if (slab + 1 == slabs) {  // chunk complete
#pragma unroll
            for (int j = 0; j < RW; ++j) {
                const uint32_t row = (chunk * RW + j) * n_waves + wid;
                const float v = wave_total(acc[j]);
                acc[j] = 0.0f;
                if (lane == 63 && row < n) y[row] = v;
            }
        }
    };

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

template <int RW, int HX>
void launch_hx(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, size_t lds, uint32_t waves,
               hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q3_b1<RW, HX>), 160 * 1024);
    hipLaunchKernelGGL((gemv_q3_b1<RW, HX>), dim3((waves + kWaves - 1) / kWaves), dim3(kWaves * 64), lds, stream, w, n, k,
                       x, y);
}

template <int RW>
void launch_rw(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, size_t lds, uint32_t waves,
               hipStream_t stream) {
    if (k <= 2048) launch_hx<RW, 1>(w, n, k, x, y, lds, waves, stream);
    else if (k <= 4096) launch_hx<RW, 2>(w, n, k, x, y, lds, waves, stream);
    else launch_hx<RW, 3>(w, n, k, x, y, lds, waves, stream);
}

}  // namespace

size_t gemv_q3_lds_bytes(uint32_t k) { return static_cast<size_t>(k / kBlockWeights) * kXPitch * 4; }

void launch_gemv_q3_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream) {
    const size_t lds = gemv_q3_lds_bytes(k);
    uint32_t wg_per_cu = static_cast<uint32_t>((160 * 1024) / (lds + 512));
    wg_per_cu = wg_per_cu > 4 ? 4 : wg_per_cu < 1 ? 1 : wg_per_cu;
    const uint32_t max_waves = 256 * wg_per_cu * kWaves;
    uint32_t rw = (n + max_waves - 1) / max_waves;
    uint32_t waves;
    if (rw <= 4) {
        waves = (n + rw - 1) / rw;  // every wave resident, one chunk each
    } else {
        waves = max_waves;          // persistent waves over many chunks
        rw = 4;
    }
    switch (rw) {
        case 1: launch_rw<1>(w, n, k, x, y, lds, waves, stream); break;
        case 2: launch_rw<2>(w, n, k, x, y, lds, waves, stream); break;
        case 3: launch_rw<3>(w, n, k, x, y, lds, waves, stream); break;
        default: launch_rw<4>(w, n, k, x, y, lds, waves, stream); break;
    }
}

}  // namespace lq4
