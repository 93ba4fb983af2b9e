// Q8_0 sibling of the batch-1 decode GEMV:  y[n] = sum_k W[n,k] * x[k]  over 34-byte blocks
// [u16 f16 scale d][32 x i8], w = q * d  (block layout forward/metal_qwen35.rs:2310-2346,
// arithmetic of gemv_q8_decode, shaders/qwen35.metal:133-190: per block sum_i f32(q_i) * x_i,
// then times f32(d), all f32).
//
// Same work layout as the Q4 kernel: lane l owns block 64 s + l of every row its wave
// processes, so a wave reads 2176 contiguous bytes per row and slab (blocks are only 2-byte
// aligned; the vector memory path takes unaligned 16-byte loads).
// Arithmetic: the weight bytes are never converted.  The 32 activations of a block are staged once per
// workgroup as 23-bit fixed point, t = rint(x * 2^22 / S) with S the power of two above the block's largest
// magnitude (the accuracy of an f32 at that magnitude, the range of f32), cut into three signed bytes
// t = b0 + 256 b1 + 65536 b2, and v_dot4_i32_i8 multiplies four weight bytes with four activation bytes and
// adds the products exactly: 24 dot instructions per block and row instead of 32 conversions and 32 FMAs.
// The three integer sums (each below 2^19) are joined in f32.
// Waves are persistent over chunks of RW rows; the next unit's blocks are in flight while the
// current one is consumed.
#include "lq4_b1_dev.hpp"

#include <type_traits>

namespace lq4 {

namespace {

constexpr int kWaves = 4;
constexpr int kXPitch = 36;  // dwords of LDS per block of x: byte plane p of weight dword w at 3 w + p (24 dwords),
                             // S * 2^-22 at 33 (16-byte lane reads at stride 144 B are conflict-free)
constexpr int kPlanes = 3;
constexpr int kQ8BlockBytes = 34;

struct __attribute__((packed, aligned(2))) Q8BlockRaw {
    uint16_t d;     // f16 scale
    uint32_t q[8];  // 32 x i8, weight i in byte i
};

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

// sum_i q_i * t_i over one block, t the block's fixed-point activations
__device__ __forceinline__ float block_dot(const uint32_t (&q)[8], const uint32_t (&xn)[8 * kPlanes]) {
    int32_t part[kPlanes] = {0, 0, 0};
#pragma unroll
    for (int w = 0; w < 8; ++w)
#pragma unroll
        for (int p = 0; p < kPlanes; ++p)
            part[p] = __builtin_amdgcn_sdot4(static_cast<int32_t>(q[w]), static_cast<int32_t>(xn[kPlanes * w + p]), part[p], false);
    return fmaf(static_cast<float>(part[2]), 65536.0f, fmaf(static_cast<float>(part[1]), 256.0f, static_cast<float>(part[0])));
}

// Chunk c of wave `wid` holds rows (c * RW + j) * n_waves + wid, j < RW; a unit is one
// (chunk, slab of 64 blocks).  Dynamic LDS: (K/32) * kXPitch dwords.
// HX: 8-activation units per thread requested ahead of the weights (all of K up to 2048 * HX).
template <int RW, int HX>
__global__ __launch_bounds__(kWaves * 64) void gemv_q8_b1(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                          const float* __restrict__ x, float* __restrict__ y) {
    extern __shared__ __attribute__((aligned(16))) uint32_t xs[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t nb = k / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ8BlockBytes;
    const uint32_t slabs = (nb + 63) / 64;
    const uint32_t n_waves = gridDim.x * kWaves;
    const uint32_t wid = __builtin_amdgcn_readfirstlane(blockIdx.x * kWaves + (tid >> 6));
    const uint32_t first = wid < n ? n - wid : 0;
    const uint32_t chunks = (first + n_waves * RW - 1) / (n_waves * RW);
    const uint32_t units = chunks * slabs;

    auto load_unit = [&](Q8BlockRaw (&buf)[RW], uint32_t u) {
        const uint32_t chunk = u / slabs, slab = u - chunk * slabs;
        uint32_t blk = slab * 64 + lane;
        if (blk >= nb) blk = nb - 1;
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            uint32_t row = (chunk * RW + j) * n_waves + wid;
            if (row >= n) row = n - 1;
            buf[j] = *reinterpret_cast<const Q8BlockRaw*>(w + row * row_bytes + blk * static_cast<uint32_t>(kQ8BlockBytes));
        }
    };

    // ---- stage x: thread g handles 8 activations of block g / 4 -----------------------------
    auto stage = [&](uint32_t g, const float4 a, const float4 b, bool store) {
        const uint32_t blk = g >> 2, j = g & 3;
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        float sx = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
        float m = fmaxf(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))),
                        fmaxf(fmaxf(fabsf(v[4]), fabsf(v[5])), fmaxf(fabsf(v[6]), fabsf(v[7]))));
        sx = dpp_add<0xB1>(sx);  // the 4 threads of a block are 4 adjacent lanes: quad butterflies
        sx = dpp_add<0x4E>(sx);
        m = b1::dpp_max_quad<0xB1>(m);
        m = b1::dpp_max_quad<0x4E>(m);
        // S = 2^(e - 126), the power of two above the block's largest magnitude (blocks below 2^-103 share that
        // scale, so S * 2^-22 stays a normal number); 2^22 / S and S * 2^-22 are exact
        uint32_t e = __builtin_bit_cast(uint32_t, m) >> 23;
        e = e < 23u ? 23u : e > 254u ? 254u : e;
        const float to_fixed = __builtin_bit_cast(float, (275u - e) << 23);
        float scale = __builtin_bit_cast(float, (e - 21u) << 23);
        // an infinite or NaN activation (or a sum that overflows) reaches every row, as it does in f32 arithmetic
        if (!(fabsf(sx) <= 3.402823466e38f)) scale = __builtin_nanf("");
        // t = rint(v * to_fixed), rounded to nearest even by the addition of 1.5 * 2^23 itself; its balanced
        // signed bytes are the low bytes of t, (t + 128) >> 8 and ((t + 128) >> 8) + 128 >> 8
        uint32_t digit[kPlanes][8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int32_t t0 = static_cast<int32_t>(__builtin_bit_cast(uint32_t, fmaf(v[i], to_fixed, 12582912.0f)) - 0x4B400000u);
            const int32_t t1 = (t0 + 128) >> 8;
            const int32_t t2 = (t1 + 128) >> 8;
            digit[0][i] = static_cast<uint32_t>(t0);
            digit[1][i] = static_cast<uint32_t>(t1);
            digit[2][i] = static_cast<uint32_t>(t2);
        }
        uint32_t out[2 * kPlanes];  // [weight dword 2j, 2j + 1][plane]
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int p = 0; p < kPlanes; ++p) {
                const uint32_t lo = b1::perm(digit[p][4 * h + 1], digit[p][4 * h + 0], 0x0c0c0400u);
                const uint32_t hi = b1::perm(digit[p][4 * h + 3], digit[p][4 * h + 2], 0x0c0c0400u);
                out[kPlanes * h + p] = b1::perm(hi, lo, 0x05040100u);
            }
        if (store) {
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            u32x2* dst = reinterpret_cast<u32x2*>(&xs[blk * kXPitch + 2 * kPlanes * j]);
            dst[0] = u32x2{out[0], out[1]};
            dst[1] = u32x2{out[2], out[3]};
            dst[2] = u32x2{out[4], out[5]};
            if (j == 0) xs[blk * kXPitch + 33] = __builtin_bit_cast(uint32_t, scale);
        }
    };

    // The first activations of every thread are requested before any weight (clamped addresses, no
    // branch): loads return in order, so behind the weight prefetch their staging, and the barrier
    // after it, would wait until the first weights have crossed from HBM.
    uint32_t gx[HX];
    float4 xa[HX], xb[HX];
#pragma unroll
    for (int i = 0; i < HX; ++i) {
        const uint32_t g = tid + i * kWaves * 64;
        gx[i] = g < nb * 4 ? g : 0;
        const float4* xp = reinterpret_cast<const float4*>(x + (gx[i] >> 2) * kBlockWeights + (gx[i] & 3) * 8);
        xa[i] = xp[0];
        xb[i] = xp[1];
    }

    Q8BlockRaw buf_a[RW], buf_b[RW];
    load_unit(buf_a, 0);  // (a wave without rows re-reads the last row; it stores nothing)
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads

#pragma unroll
    for (int i = 0; i < HX; ++i) stage(gx[i], xa[i], xb[i], tid + i * kWaves * 64 < nb * 4);
    for (uint32_t g = tid + HX * kWaves * 64; g < nb * 4; g += kWaves * 64) {
        const float4* xp = reinterpret_cast<const float4*>(x + (g >> 2) * kBlockWeights + (g & 3) * 8);
        stage(g, xp[0], xp[1], true);
    }
    __syncthreads();

    float acc[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) acc[j] = 0.0f;

    // `prefetch` is a compile-time flag: behind a run-time condition the compiler would have to wait
    // for most of the just-issued next unit before it may use the current one.
    auto process = [&](auto prefetch, Q8BlockRaw (&cur)[RW], Q8BlockRaw (&nxt)[RW], uint32_t u) {
        const uint32_t chunk = u / slabs, slab = u - chunk * slabs;
        if constexpr (decltype(prefetch)::value) load_unit(nxt, u + 1);
        const uint32_t blk_raw = slab * 64 + lane;
        const bool live = blk_raw < nb;
        const uint32_t blk = live ? blk_raw : nb - 1;
        uint32_t xn[8 * kPlanes];
        const uint4* xsrc = reinterpret_cast<const uint4*>(&xs[blk * kXPitch]);
#pragma unroll
        for (int i = 0; i < 2 * kPlanes; ++i) {
            const uint4 v = xsrc[i];
            xn[4 * i + 0] = v.x; xn[4 * i + 1] = v.y; xn[4 * i + 2] = v.z; xn[4 * i + 3] = v.w;
        }
        const float scale_x = __builtin_bit_cast(float, xs[blk * kXPitch + 33]);
#pragma unroll
        for (int j = 0; j < RW; ++j) {
            const float p = block_dot(cur[j].q, xn);
            const float d = live ? f16_bits_to_f32(cur[j].d) : 0.0f;
            acc[j] = fmaf(d * p, scale_x, acc[j]);
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
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q8_b1<RW, HX>), 160 * 1024);
    hipLaunchKernelGGL((gemv_q8_b1<RW, HX>), dim3((waves + kWaves - 1) / kWaves), dim3(kWaves * 64), lds, stream, w, n, k,
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

size_t gemv_q8_lds_bytes(uint32_t k) { return static_cast<size_t>(k / kBlockWeights) * kXPitch * 4; }

void launch_gemv_q8_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream) {
    const size_t lds = gemv_q8_lds_bytes(k);
    uint32_t wg_per_cu = static_cast<uint32_t>((160 * 1024) / (lds + 512));
    wg_per_cu = wg_per_cu > 4 ? 4 : wg_per_cu < 1 ? 1 : wg_per_cu;
    const uint32_t max_waves = 256 * wg_per_cu * kWaves;
    uint32_t rw = (n + max_waves - 1) / max_waves;
    uint32_t waves;
    if (rw <= 4) {
        waves = (n + rw - 1) / rw;  // every wave resident, one chunk each
    } else {
        waves = max_waves;          // persistent waves over many chunks
        rw = 2;
    }
    switch (rw) {
        case 1: launch_rw<1>(w, n, k, x, y, lds, waves, stream); break;
        case 2: launch_rw<2>(w, n, k, x, y, lds, waves, stream); break;
        case 3: launch_rw<3>(w, n, k, x, y, lds, waves, stream); break;
        default: launch_rw<4>(w, n, k, x, y, lds, waves, stream); break;
    }
}

}  // namespace lq4
