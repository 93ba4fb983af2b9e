// Decode GEMV for 1..8 activation rows over native Q4 blocks, on the matrix cores:
//   y[b, n] = sum_k W[n, k] * x[b, k],  b < batch.
//
// The kernel is HBM-bound by design; everything below exists to keep the cores' side of
// the work (unpack, multiply, scale) well under the time the bytes take to arrive.
//
// Instruction.  v_mfma_f32_4x4x4_16B_f16 multiplies 16 independent 4x4x4 problems, one per
// group of four lanes.  Lane 4g+j supplies B[:, j] (4 values) and A[j, :] (4 values) of
// group g and receives D[0..3, j] = sum_k A[i, k] * B[k, j].  Here B[:, j] are 4 weights of
// the lane's own block and A[i, :] is the matching slice of activation column i, so a lane
// gets the dot products of ITS weights with up to four activation columns; the other three
// lanes of the group hold the same block position of three other weight rows.  Eight such
// instructions cover a 32-weight block.
//
// Mapping.  Lane 4g+j of a wave owns block 16*s + g (s = step along K) of weight rows
// 4t + j, t < T: one contiguous 20-byte block per row per step (dwordx4 + dword), 16
// consecutive blocks (320 contiguous bytes) per row per wave-step, nothing fetched twice.
// The waves of a workgroup split K (KS slices) and row groups (4/KS); partial sums meet in
// LDS.  Activations are staged once per workgroup in LDS as f16, already in the order the
// unpack yields.
//
// Unpack.  A masked dword IS a pair of f16 subnormals: q & 0x000F000F = (n0, n4) * 2^-24 and
// q & 0x00F000F0 = (n1, n5) * 2^-20 (the matrix cores honour f16 subnormals), so five VALU ops
// turn 8 nibbles into 8 exact f16 operands; activations paired with the 2^-20 form are
// pre-scaled by 2^-4, and the block scale absorbs 2^24.  Per block, in f32:
//   y += (d * 2^24) * P + b * sum_k x_k      (P from the matrix core; the bias-factored form
//   of the reference kernel, shaders/qwen35.metal:838-847).
//
// Precision.  For batch <= 2 every f32 activation is split x = hi + lo/2048 (two f16 columns),
// products are exact and the result tracks an f32 GEMV (~1e-6), as the reference's m == 1 kernel
// does.  For batch >= 3 activations are rounded to f16 once, as the reference's m > 1 tiled
// kernel does (shaders/gemm_q4_tiled.metal:45-48).  Activations must be finite and within the
// f16 range (|x| < 65504).
#include "lq4_internal.hpp"

namespace lq4 {

namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr float kLoScale = 2048.0f;
constexpr float kTwo24 = 16777216.0f;

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

__device__ __forceinline__ uint32_t pack_h2(_Float16 a, _Float16 b) {
    const half2v h = {a, b};
    return __builtin_bit_cast(uint32_t, h);
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
    return v + __builtin_bit_cast(float, moved);
}

// LDS bytes per block of K: `ncols` columns of 32 f16 (64 B each) followed by the per-row
// sums of x (one f32 per activation row, padded to 16 B).
__host__ __device__ constexpr uint32_t x_pitch_bytes(int ncols, int batch) {
    return static_cast<uint32_t>(ncols) * 64u + 16u * static_cast<uint32_t>((batch + 3) / 4);
}

// 8 consecutive activations -> the operand order of one packed dword:
// [x0, x4, x1/16, x5/16 | x2, x6, x3/16, x7/16]  (first / second 4x4x4 step of the dword).
template <bool HILO>
__device__ __forceinline__ void convert_x8(const float4 a, const float4 b, uint4& hi, uint4& lo, float& sum_x) {
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    _Float16 h[8], l[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float s = (i & 1) ? v[i] * 0.0625f : v[i];
        h[i] = static_cast<_Float16>(s);
        l[i] = HILO ? static_cast<_Float16>((s - static_cast<float>(h[i])) * kLoScale) : static_cast<_Float16>(0.0f);
    }
    hi.x = pack_h2(h[0], h[4]); hi.y = pack_h2(h[1], h[5]); hi.z = pack_h2(h[2], h[6]); hi.w = pack_h2(h[3], h[7]);
    lo.x = pack_h2(l[0], l[4]); lo.y = pack_h2(l[1], l[5]); lo.z = pack_h2(l[2], l[6]); lo.w = pack_h2(l[3], l[7]);
    sum_x = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
}

struct GemvArgs {
    const uint8_t* w;
    const float* x;
    float* y;
    uint32_t n, k, batch, x_stride, y_stride;
    LoraEpilogue lora;
    // Elementwise steps around the product, per activation row (the batch form of the one-token
    // kernel's GemvFusion): base, delta and residual_out are [batch, K] rows, x for kSiluMul is
    // [batch, 2K] rows of [gate | up] (x_stride apart), residual and copy_dst are [batch, N] rows
    // (y_stride apart).  kPlain / kStore: the plain product.
    GemvFusion fz;
};

// NSETS: groups of four activation columns (1 or 2).  HILO: two columns per activation row.
// T: weight-row tiles (of 4 rows) per wave.  KS: slices of K per workgroup (1, 2 or 4).
// WAVES: waves per workgroup (4 or 8), all served by one staged copy of the activations.
// Workgroups are persistent: workgroup g handles row groups g, g + gridDim.x, ... (a row group
// is 4*T*(WAVES/KS) rows) with the activations staged once.  For one wave the work is a list of
// units (row group, step); unit u+1 is in flight while unit u is consumed.
template <int NSETS, bool HILO, int T, int KS, bool LONG, int WAVES, bool DEEP>
__global__ __launch_bounds__(64 * WAVES) void gemv_q4_mfma(GemvArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int kThreads = 64 * WAVES;
    constexpr int RS = WAVES / KS;  // row sub-groups per workgroup
    constexpr int NCOLS = 4 * NSETS;
    constexpr uint32_t kRowsPerIter = 4 * T * RS;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 2;   // block within the step
    const int j = lane & 3;    // weight row within the tile / activation column within a set
    const uint32_t nb = p.k / kBlockWeights;
    const uint32_t nsteps = (nb + 15) / 16;
    const uint32_t batch = p.batch;
    const int ncols = HILO ? 2 * static_cast<int>(batch) : static_cast<int>(batch);
    const uint32_t pitch = x_pitch_bytes(ncols, batch);
    // LDS is addressed in 16-byte units so every vector access is provably aligned
    uint4* const xs16 = reinterpret_cast<uint4*>(smem);
    const uint32_t pitch16 = pitch / 16;
    uint4* const zero_region = xs16 + nb * pitch16;               // 64 B of zeros
    float* red = reinterpret_cast<float*>(zero_region + 4);       // [2][WAVES][T][NCOLS][4]
    constexpr int kRedFloats = WAVES * T * NCOLS * 4;

    const int ks = wave % KS, rs = wave / KS;
    const uint32_t n_groups = (p.n + kRowsPerIter - 1) / kRowsPerIter;
    const uint32_t iters = (n_groups - blockIdx.x + gridDim.x - 1) / gridDim.x;  // >= 1
    const uint32_t n_local = static_cast<uint32_t>(ks) < nsteps ? (nsteps - ks + KS - 1) / KS : 0;
    const uint32_t units = iters * n_local;
    auto first_row = [&](uint32_t it) { return ((blockIdx.x + it * gridDim.x) * RS + rs) * (4 * T); };

    // ---- the first activations are requested before any weight, so they can be waited on alone
    // (loads return in order: behind the weight prefetch their staging would wait for the weights).
    // One (row, item) pair per thread, or a whole round of four with eight activation columns, whose
    // kernels have the registers to spare at the occupancy their staged activations allow.
    const uint32_t items = nb * 4;  // (block, dword) pairs per activation row
    const uint32_t total_items = batch * items;
    constexpr int kHoist = NSETS == 2 ? 4 : 1;
    float4 hva[kHoist], hvb[kHoist];
    uint32_t hrow[kHoist], hitem[kHoist];
#pragma unroll
    for (int i = 0; i < kHoist; ++i) {
        const uint32_t w = tid + i * kThreads;
        const uint32_t wc = w < total_items ? w : 0;
        hrow[i] = wc / items;
        hitem[i] = wc - hrow[i] * items;
        if (p.fz.prologue == GemvFusion::kPlain) {  // uniform; the fused prologues load everything below
            const float4* xp = reinterpret_cast<const float4*>(p.x + static_cast<size_t>(hrow[i]) * p.x_stride +
                                                               (hitem[i] >> 2) * kBlockWeights + (hitem[i] & 3) * 8);
            hva[i] = xp[0];
            hvb[i] = xp[1];
        } else {
            hva[i] = hvb[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    }

    // Loads unit u.  Blocks past the end of a row and rows past N re-read a valid block; their
    // contribution is zeroed or dropped later.
    auto load_unit = [&](Q4BlockRaw (&buf)[T], uint32_t u) {
        const uint32_t it = n_local ? u / n_local : 0, q = u - it * n_local;
        uint32_t blk = (ks + q * KS) * 16 + g;
        if (blk >= nb) blk = nb - 1;
        const uint32_t row0 = first_row(it);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            uint32_t row = row0 + 4 * t + j;
            if (row >= p.n) row = p.n - 1;
            buf[t] = *reinterpret_cast<const Q4BlockRaw*>(reinterpret_cast<const uint32_t*>(p.w) +
                                                          static_cast<size_t>(row) * (nb * 5) + blk * 5);
        }
    };

    // Unit buffers in registers.  DEEP: a ring of four, three units in flight while one is consumed; else two, the
    // next unit in flight while one is consumed.  The shallow form is the faster one except on very long rows
    // (measured at 2 / 4 / 8 rows: 12288 x 2048 8.0 / 7.8 / - -> 6.3 / 7.4 / - us, 6144 x 2048 at 2 rows 6.8 -> 5.0,
    // 2048 x 6144 5.8 / 6.6 / 8.4 -> 5.8 / 6.4 / 8.0, 17408 x 5120 18.1 / 20.4 / 24.2 -> 17.0 / 18.6 / 24.2, 8192 x 8192
    // 13.9 / 15.2 / 19.2 -> 13.2 / 14.5 / 18.0; but 5120 x 17408 19.6 / 21.5 -> 21.4 / 23.1): what a CU asks for beyond
    // its share of the memory system queues in front of the activations its workgroups' staging waits for.
    Q4BlockRaw buf_a[T], buf_b[T], buf_c[T], buf_d[T];
    load_unit(buf_a, 0);
    if constexpr (DEEP) {
        load_unit(buf_b, units > 1 ? 1 : 0);
        load_unit(buf_c, units > 2 ? 2 : 0);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads

    // ---- stage activations: one (block, dword) item = 8 values per activation row ------------
    auto stage = [&](uint32_t it, uint32_t b, const float4 va, const float4 vb, bool store) {
        const uint32_t blk = it >> 2, dw = it & 3;
        uint4 hi, lo;
        float sx;
        convert_x8<HILO>(va, vb, hi, lo, sx);
        sx = dpp_add<0xB1>(sx);  // the 4 items of a block sit in 4 adjacent lanes
        sx = dpp_add<0x4E>(sx);
        if (store) {
            uint4* base = xs16 + blk * pitch16;
            if (HILO) {
                base[(2 * b) * 4 + dw] = hi;
                base[(2 * b + 1) * 4 + dw] = lo;
            } else {
                base[b * 4 + dw] = hi;
            }
            if (dw == 0) reinterpret_cast<float*>(base + ncols * 4)[b] = sx;
        }
    };
    // The activations are produced while they are staged (the batch form of the one-token kernel's
    // prologues; shaders/qwen35.metal:2219-2249 is the reference's batched add + norm, :712-722 its
    // silu * up).  Every workgroup does this for all rows, as it stages all rows anyway.
    auto stage_fused = [&]() {
        auto unit_at = [](uint32_t it) { return (it >> 2) * kBlockWeights + (it & 3) * 8; };
        auto add4 = [](float4 a, const float4 b) {
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
            return a;
        };
        constexpr int G = 2;  // pairs in flight per thread (each is four 16-byte loads)
        if (p.fz.prologue == GemvFusion::kAddNorm) {
            // 1/rms of every row first: wave v owns rows v, v + WAVES, ...; a lane sums units lane, lane + 64, ...
            // in order, then the wave sum: the same value in every workgroup.  Workgroup 0 stores the new residual.
            float* inv_rms = red;  // [batch]: the K slices' meeting point is not in use yet
            for (uint32_t b = wave; b < batch; b += WAVES) {
                const float* bp = p.fz.base + static_cast<size_t>(b) * p.k;
                const float* dp = p.fz.delta ? p.fz.delta + static_cast<size_t>(b) * p.k : nullptr;
                float ss = 0.0f;
                for (uint32_t it0 = lane; it0 < items; it0 += 64 * 4) {
                    float4 a[4], c[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t it = it0 + 64 * i < items ? it0 + 64 * i : 0;
                        a[i] = reinterpret_cast<const float4*>(bp + unit_at(it))[0];
                        c[i] = reinterpret_cast<const float4*>(bp + unit_at(it))[1];
                        if (dp) {
                            a[i] = add4(a[i], reinterpret_cast<const float4*>(dp + unit_at(it))[0]);
                            c[i] = add4(c[i], reinterpret_cast<const float4*>(dp + unit_at(it))[1]);
                        }
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (it0 + 64 * i < items) {
                            ss += ((a[i].x * a[i].x + a[i].y * a[i].y) + (a[i].z * a[i].z + a[i].w * a[i].w)) +
                                  ((c[i].x * c[i].x + c[i].y * c[i].y) + (c[i].z * c[i].z + c[i].w * c[i].w));
                            if (blockIdx.x == 0 && p.fz.residual_out) {
                                float4* rp = reinterpret_cast<float4*>(p.fz.residual_out + static_cast<size_t>(b) * p.k + unit_at(it0 + 64 * i));
                                rp[0] = a[i];
                                rp[1] = c[i];
                            }
                        }
                    }
                }
                ss = wave_sum(ss);
                if (lane == 0) inv_rms[b] = 1.0f / sqrtf(ss / static_cast<float>(p.k) + p.fz.eps);
            }
            __syncthreads();
            for (uint32_t w0 = tid; w0 < total_items; w0 += G * kThreads) {
                float4 va[G], vb[G], ga[G], gb[G];
                uint32_t wb[G], wi[G];
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    const uint32_t w = w0 + i * kThreads;
                    const uint32_t wc = w < total_items ? w : 0;
                    wb[i] = wc / items;
                    wi[i] = wc - wb[i] * items;
                    const size_t at = static_cast<size_t>(wb[i]) * p.k + unit_at(wi[i]);
                    va[i] = reinterpret_cast<const float4*>(p.fz.base + at)[0];
                    vb[i] = reinterpret_cast<const float4*>(p.fz.base + at)[1];
                    if (p.fz.delta) {
                        va[i] = add4(va[i], reinterpret_cast<const float4*>(p.fz.delta + at)[0]);
                        vb[i] = add4(vb[i], reinterpret_cast<const float4*>(p.fz.delta + at)[1]);
                    }
                    ga[i] = reinterpret_cast<const float4*>(p.fz.gamma + unit_at(wi[i]))[0];
                    gb[i] = reinterpret_cast<const float4*>(p.fz.gamma + unit_at(wi[i]))[1];
                }
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    const float inv = inv_rms[wb[i]];
                    auto norm4 = [inv](float4 v, const float4 gm) {
                        v.x = v.x * inv * (1.0f + gm.x); v.y = v.y * inv * (1.0f + gm.y);
                        v.z = v.z * inv * (1.0f + gm.z); v.w = v.w * inv * (1.0f + gm.w);
                        return v;
                    };
                    stage(wi[i], wb[i], norm4(va[i], ga[i]), norm4(vb[i], gb[i]), w0 + i * kThreads < total_items);
                }
            }
            __syncthreads();  // inv_rms has been read by all before the meeting point is written
        } else {  // kSiluMul: silu through the hardware exp2 and reciprocal, as the one-token kernel does
            auto silu_mul = [](float gate, float u) {
                const float e = __builtin_amdgcn_exp2f(gate * -1.44269504088896340736f);
                return gate * __builtin_amdgcn_rcpf(1.0f + e) * u;
            };
            for (uint32_t w0 = tid; w0 < total_items; w0 += G * kThreads) {
                float4 ga[G], gb[G], ua[G], ub[G];
                uint32_t wb[G], wi[G];
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    const uint32_t w = w0 + i * kThreads;
                    const uint32_t wc = w < total_items ? w : 0;
                    wb[i] = wc / items;
                    wi[i] = wc - wb[i] * items;
                    const float* gp = p.x + static_cast<size_t>(wb[i]) * p.x_stride + unit_at(wi[i]);
                    ga[i] = reinterpret_cast<const float4*>(gp)[0];
                    gb[i] = reinterpret_cast<const float4*>(gp)[1];
                    ua[i] = reinterpret_cast<const float4*>(gp + p.k)[0];
                    ub[i] = reinterpret_cast<const float4*>(gp + p.k)[1];
                }
#pragma unroll
                for (int i = 0; i < G; ++i) {
                    float4 a, b;
                    a.x = silu_mul(ga[i].x, ua[i].x); a.y = silu_mul(ga[i].y, ua[i].y);
                    a.z = silu_mul(ga[i].z, ua[i].z); a.w = silu_mul(ga[i].w, ua[i].w);
                    b.x = silu_mul(gb[i].x, ub[i].x); b.y = silu_mul(gb[i].y, ub[i].y);
                    b.z = silu_mul(gb[i].z, ub[i].z); b.w = silu_mul(gb[i].w, ub[i].w);
                    stage(wi[i], wb[i], a, b, w0 + i * kThreads < total_items);
                }
            }
        }
    };
    if (p.fz.prologue != GemvFusion::kPlain) {
        stage_fused();
    } else {
#pragma unroll
    for (int i = 0; i < kHoist; ++i) stage(hitem[i], hrow[i], hva[i], hvb[i], tid + i * kThreads < total_items);
    // the remaining (row, item) pairs, four loads in flight per thread so that a batch of rows costs
    // a couple of memory round trips, not one per row
    {
        constexpr int G = 4;
        const uint32_t total = total_items;
        for (uint32_t w0 = tid + kHoist * kThreads; w0 < total; w0 += G * kThreads) {
            float4 va[G], vb[G];
            uint32_t wb[G], wi[G];
#pragma unroll
            for (int i = 0; i < G; ++i) {
                const uint32_t w = w0 + i * kThreads;
                const uint32_t wc = w < total ? w : 0;
                wb[i] = wc / items;
                wi[i] = wc - wb[i] * items;
                const float4* xp = reinterpret_cast<const float4*>(p.x + static_cast<size_t>(wb[i]) * p.x_stride +
                                                                   (wi[i] >> 2) * kBlockWeights + (wi[i] & 3) * 8);
                va[i] = xp[0];
                vb[i] = xp[1];
            }
#pragma unroll
            for (int i = 0; i < G; ++i) stage(wi[i], wb[i], va[i], vb[i], w0 + i * kThreads < total);
        }
    }
    }
    if (tid < 4) zero_region[tid] = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();

    float acc[T][NCOLS];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
        for (int c = 0; c < NCOLS; ++c) acc[t][c] = 0.0f;

    // Consumes unit u from `cur` while unit u+1 streams into `nxt`.
    auto process = [&](Q4BlockRaw (&cur)[T], Q4BlockRaw (&nxt)[T], uint32_t u) {
        // LONG streams prefetch without a condition (past the end: the last unit again), so the wait
        // for the current unit counts exactly and three units stay in flight; short streams, whose
        // units are all in flight from the start, skip the redundant loads instead
        constexpr uint32_t kAhead = DEEP ? 3 : 1;
        if (LONG) load_unit(nxt, u + kAhead < units ? u + kAhead : units - 1);
        else if (u + kAhead < units) load_unit(nxt, u + kAhead);
        const uint32_t it = u / n_local, q = u - it * n_local;
        const uint32_t blk_raw = (ks + q * KS) * 16 + g;
        const bool live = blk_raw < nb;
        const uint32_t blk = live ? blk_raw : nb - 1;
        const uint4* xb = xs16 + blk * pitch16;

        // activation operands of this lane: column 4*set + j of block `blk` (zeros past ncols)
        uint32_t a_op[NSETS][16];
#pragma unroll
        for (int set = 0; set < NSETS; ++set) {
            const int col = 4 * set + j;
            const uint4* src = col < ncols ? xb + col * 4 : zero_region;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 v = src[i];
                a_op[set][4 * i + 0] = v.x; a_op[set][4 * i + 1] = v.y;
                a_op[set][4 * i + 2] = v.z; a_op[set][4 * i + 3] = v.w;
            }
        }
        // sum of x over the block, for the column that carries the bias term of its activation row
        float sum_x[NCOLS];
#pragma unroll
        for (int c = 0; c < NCOLS; ++c) {
            const int brow = HILO ? c / 2 : c;
            const bool has = (HILO ? (c % 2 == 0) : true) && brow < static_cast<int>(batch) && live;
            sum_x[c] = has ? reinterpret_cast<const float*>(xb + ncols * 4)[brow] : 0.0f;
        }

#pragma unroll
        for (int t = 0; t < T; ++t) {
            float4v prod[NSETS];
#pragma unroll
            for (int set = 0; set < NSETS; ++set) prod[set] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int dw = 0; dw < 4; ++dw) {
                const uint32_t qd = cur[t].q[dw];
                const uint32_t q8 = qd >> 8;
                const uint32_t w0 = qd & 0x000F000Fu, w1 = qd & 0x00F000F0u;
                const uint32_t w2 = q8 & 0x000F000Fu, w3 = q8 & 0x00F000F0u;
                const half4 b01 = __builtin_bit_cast(half4, uint2{w0, w1});
                const half4 b23 = __builtin_bit_cast(half4, uint2{w2, w3});
#pragma unroll
                for (int set = 0; set < NSETS; ++set) {
                    const half4 a01 = __builtin_bit_cast(half4, uint2{a_op[set][4 * dw + 0], a_op[set][4 * dw + 1]});
                    const half4 a23 = __builtin_bit_cast(half4, uint2{a_op[set][4 * dw + 2], a_op[set][4 * dw + 3]});
                    prod[set] = __builtin_amdgcn_mfma_f32_4x4x4f16(a01, b01, prod[set], 0, 0, 0);
                    prod[set] = __builtin_amdgcn_mfma_f32_4x4x4f16(a23, b23, prod[set], 0, 0, 0);
                }
            }
            float d = f16_bits_to_f32(cur[t].sb & 0xffffu) * kTwo24;
            const float bias = f16_bits_to_f32(cur[t].sb >> 16);
            if (!live) d = 0.0f;
#pragma unroll
            for (int c = 0; c < NCOLS; ++c)
                acc[t][c] = fmaf(d, prod[c / 4][c % 4], fmaf(bias, sum_x[c], acc[t][c]));
        }
    };

    // Row group finished for this wave: sum over the 16 blocks of a step (lanes with equal j),
    // meet the other K slices in LDS, and let the slice-0 wave store.
    auto finish = [&](uint32_t it) {
        // LoRA delta, spread over the 16 lanes that share a weight row: lane group g adds
        // scale * B[row, r] * t[brow, r] for r = g, g + 16, ... to its partial sums (slice-0 waves
        // only, so it is counted once); the reduction below then sums it with everything else.
        if (p.lora.rank && ks == 0) {
            const uint32_t lrow0 = first_row(it);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                uint32_t row = lrow0 + 4 * t + j;
                if (row >= p.n) row = p.n - 1;
                for (uint32_t r = g; r < p.lora.rank; r += 16) {
                    const size_t bi = static_cast<size_t>(row) * p.lora.rank + r;
                    const float bv = p.lora.scale *
                                     (p.lora.b_is_f16 ? static_cast<float>(static_cast<const _Float16*>(p.lora.b)[bi])
                                                      : static_cast<const float*>(p.lora.b)[bi]);
#pragma unroll
                    for (int c = 0; c < NCOLS; ++c) {
                        const int brow = HILO ? c / 2 : c;
                        if ((HILO && (c & 1)) || brow >= static_cast<int>(batch)) continue;
                        acc[t][c] = fmaf(bv, p.lora.t[brow * p.lora.rank + r], acc[t][c]);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int c = 0; c < NCOLS; ++c) {
                float v = acc[t][c];
                acc[t][c] = 0.0f;
                v = dpp_add<0x124>(v);  // row_ror:4
                v = dpp_add<0x128>(v);  // row_ror:8 -> sum over the row's lanes with this j
                v = sum_over_rows(v);
                if (KS > 1 && lane < 4) red[(it & 1) * kRedFloats + ((wave * T + t) * NCOLS + c) * 4 + lane] = v;
                if (KS == 1) acc[t][c] = v;  // reused below as the total
            }
        if (KS > 1) __syncthreads();
        if (ks == 0 && lane < 4) {
            const uint32_t row0 = first_row(it);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const uint32_t row = row0 + 4 * t + lane;
                float tot[NCOLS];
#pragma unroll
                for (int c = 0; c < NCOLS; ++c) {
                    float v = KS == 1 ? acc[t][c] : 0.0f;
                    if (KS > 1)
                        for (int o = 0; o < KS; ++o)
                            v += red[(it & 1) * kRedFloats + (((wave + o) * T + t) * NCOLS + c) * 4 + lane];
                    tot[c] = v;
                }
                if (row < p.n) {
#pragma unroll
                    for (int c = 0; c < NCOLS; ++c) {
                        const int brow = HILO ? c / 2 : c;
                        if ((HILO && (c & 1)) || brow >= static_cast<int>(batch)) continue;
                        const float v = HILO ? fmaf(tot[c + (HILO ? 1 : 0)], 1.0f / kLoScale, tot[c]) : tot[c];
                        const size_t at = static_cast<size_t>(brow) * p.y_stride + row;
                        if (p.fz.epilogue == GemvFusion::kAddResidual) {
                            const float r = p.fz.residual[at] + v;
                            p.fz.residual[at] = r;
                            if (p.fz.copy_dst) p.fz.copy_dst[at] = r;
                            if (p.y) p.y[at] = v;
                        } else {
                            p.y[at] = v;
                        }
                    }
                }
            }
        }
        if (KS == 1) {
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int c = 0; c < NCOLS; ++c) acc[t][c] = 0.0f;
        }
    };

    if (n_local == 0) {  // more K slices than steps: this wave only takes part in the barriers
        for (uint32_t it = 0; it < iters; ++it) finish(it);
        return;
    }
    // the buffers rotate roles every unit, so no block is ever copied between registers
    uint32_t q = 0, it = 0;
    if constexpr (!DEEP) {
        for (uint32_t u = 0; u < units; u += 2) {
            process(buf_a, buf_b, u);
            if (++q == n_local) { finish(it++); q = 0; }
            if (u + 1 >= units) break;
            process(buf_b, buf_a, u + 1);
            if (++q == n_local) { finish(it++); q = 0; }
        }
        return;
    }
    for (uint32_t u = 0; u < units; u += 4) {
        process(buf_a, buf_d, u);
        if (++q == n_local) { finish(it++); q = 0; }
        if (u + 1 >= units) break;
        process(buf_b, buf_a, u + 1);
        if (++q == n_local) { finish(it++); q = 0; }
        if (u + 2 >= units) break;
        process(buf_c, buf_b, u + 2);
        if (++q == n_local) { finish(it++); q = 0; }
        if (u + 3 >= units) break;
        process(buf_d, buf_c, u + 3);
        if (++q == n_local) { finish(it++); q = 0; }
    }
}

template <int NSETS, bool HILO, int T, int KS, bool LONG, int WAVES, bool DEEP>
void launch_deep(const GemvArgs& a, size_t lds, uint32_t wgs, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q4_mfma<NSETS, HILO, T, KS, LONG, WAVES, DEEP>), 160 * 1024);
    hipLaunchKernelGGL((gemv_q4_mfma<NSETS, HILO, T, KS, LONG, WAVES, DEEP>), dim3(wgs), dim3(64 * WAVES), lds, stream, a);
}

// the ring of four only for very long rows, which come with eight-wave workgroups (one staged copy per CU)
template <int NSETS, bool HILO, int T, int KS, bool LONG, int WAVES>
void launch_long(const GemvArgs& a, size_t lds, uint32_t wgs, hipStream_t stream) {
    if constexpr (WAVES == 8 && LONG) {
        if (a.k >= 12288) return launch_deep<NSETS, HILO, T, KS, LONG, WAVES, true>(a, lds, wgs, stream);
    }
    launch_deep<NSETS, HILO, T, KS, LONG, WAVES, false>(a, lds, wgs, stream);
}

template <int NSETS, bool HILO, int T, int KS, int WAVES>
void launch_cfg(const GemvArgs& a, size_t lds, uint32_t max_wgs, hipStream_t stream) {
    constexpr uint32_t rows_per_iter = 4 * T * (WAVES / KS);
    const uint32_t groups = (a.n + rows_per_iter - 1) / rows_per_iter;
    // every workgroup gets the same number of row groups, to within one
    const uint32_t iters = (groups + max_wgs - 1) / max_wgs;
    const uint32_t wgs = (groups + iters - 1) / iters;
    const uint32_t nsteps = (a.k / kBlockWeights + 15) / 16;
    const uint32_t units = iters * ((nsteps + KS - 1) / KS);  // per wave
    if (units >= 8) launch_long<NSETS, HILO, T, KS, true, WAVES>(a, lds, wgs, stream);
    else launch_long<NSETS, HILO, T, KS, false, WAVES>(a, lds, wgs, stream);
}

template <int NSETS, bool HILO>
void launch_shape(const GemvArgs& a, size_t lds, uint32_t t, uint32_t ks, uint32_t waves, uint32_t max_wgs,
                  hipStream_t stream) {
#define LQ4_CASE(T_, KS_, W_) \
    if (t == T_ && ks == KS_ && waves == W_) return launch_cfg<NSETS, HILO, T_, KS_, W_>(a, lds, max_wgs, stream)
    LQ4_CASE(1, 4, 4); LQ4_CASE(1, 2, 4); LQ4_CASE(1, 1, 4);
    LQ4_CASE(2, 4, 4); LQ4_CASE(2, 2, 4); LQ4_CASE(2, 1, 4);
    LQ4_CASE(4, 4, 4); LQ4_CASE(4, 2, 4); LQ4_CASE(4, 1, 4);
    LQ4_CASE(1, 4, 8); LQ4_CASE(1, 2, 8); LQ4_CASE(1, 1, 8);
    LQ4_CASE(2, 4, 8); LQ4_CASE(2, 2, 8); LQ4_CASE(2, 1, 8);
#undef LQ4_CASE
}

}  // namespace

// the K slices' meeting point: [2][waves][T <= 4][columns <= 8][4] floats
constexpr size_t kRedBytes4 = 2 * 4 * 4 * 8 * 4 * sizeof(float);
constexpr size_t kRedBytes8 = 2 * 8 * 2 * 8 * 4 * sizeof(float);  // eight waves come with T <= 2
static_assert(kRedBytes8 <= kRedBytes4, "the eight-wave kernels must fit the LDS size the routing was told");

size_t gemv_mfma_lds_bytes(uint32_t k, uint32_t batch) {
    const bool hilo = batch <= 2;
    const int ncols = hilo ? 2 * batch : batch;
    return static_cast<size_t>(k / kBlockWeights) * x_pitch_bytes(ncols, batch) + 64 +
           kRedBytes4;
}

void launch_gemv_mfma(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride,
                      uint32_t batch, float* y, uint32_t y_stride, const LoraEpilogue& lora,
                      hipStream_t stream, const GemvFusion* fusion) {
    GemvArgs a{w, x, y, n, k, batch, x_stride, y_stride, lora, fusion ? *fusion : GemvFusion{}};
    const size_t lds = gemv_mfma_lds_bytes(k, batch);
    const uint32_t nsteps = (k / kBlockWeights + 15) / 16;
    // resident workgroups per CU: up to 8 (32 waves, what the T = 1 kernels' 64 registers allow)
    // unless the staged activations leave room for fewer
    uint32_t wg_per_cu = static_cast<uint32_t>((160 * 1024) / (lds + 1024));
    wg_per_cu = wg_per_cu > 8 ? 8 : wg_per_cu < 1 ? 1 : wg_per_cu;
    const uint32_t max_wgs = 256 * wg_per_cu;
    // K slices per workgroup: none when the rows alone give about 3 workgroups per CU (no LDS
    // meeting point, no barrier per row group); otherwise split K as far as its steps allow
    // Waves per workgroup: eight where the staged activations leave room for one workgroup per CU
    // only (one copy then serves twice the waves: 17408 x 5120 at 8 rows 27.2 -> 23.4 us, 5120 x 17408
    // at 4 rows 24.9 -> 21.3), for matrices of at most 2048 rows, whose rows are too few to go round
    // (2048 x 2048 at 8 rows 6.0 -> 4.9 us), and for one or two rows of a matrix below 2^25 weights
    // (2048 x 6144 at 2 rows 7.3 -> 5.8 us).  Elsewhere the wider workgroup was measured slower
    // (12288 x 2048 at 4 rows 7.5 -> 8.9 us): fewer, larger workgroups balance worse over the CUs.
    const uint64_t weights = static_cast<uint64_t>(n) * k;
    const uint32_t waves = wg_per_cu == 1 || n <= 2048 || (batch <= 2 && weights < (1ull << 25)) ? 8 : 4;
    uint32_t ks = 1;
    while (ks < 4 && ks * 2 <= nsteps && (n + 4 * waves / ks - 1) / (4 * waves / ks) < 768) ks *= 2;
    // row tiles per wave: enough blocks in flight per CU to cover HBM latency (about 40 KB), but
    // never so many that fewer than two workgroups per CU remain
    uint32_t t = wg_per_cu >= 4 ? 1 : wg_per_cu >= 2 ? 2 : 4;
    while (t > 1 && (n + 4 * t * (waves / ks) - 1) / (4 * t * (waves / ks)) < 512) t >>= 1;
    if (waves == 8 && t > 2) t = 2;
    if (batch <= 2) {
        launch_shape<1, true>(a, lds, t, ks, waves, max_wgs, stream);
    } else if (batch <= 4) {
        launch_shape<1, false>(a, lds, t, ks, waves, max_wgs, stream);
    } else {
        launch_shape<2, false>(a, lds, t, ks, waves, max_wgs, stream);
    }
}

}  // namespace lq4
