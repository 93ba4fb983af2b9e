// Decode GEMV for up to eight activation rows on the integer matrix cores:
//   y[b, n] = sum_k W[n, k] * x[b, k],  b < batch <= 8.
//
// Instruction.  v_mfma_i32_16x16x32_i8 multiplies a 16 x 32 by a 32 x 16 matrix of signed bytes into 16 x 16 32-bit
// sums.  K = 32 is exactly one Q4 block, so one instruction forms the integer dot products of one block of 16 weight
// rows with 16 activation columns, and the block's scale and bias are applied to its result in f32 afterwards.
//   B operand (32 x 16): the weights.  Lane l supplies column n = l % 16 (a weight row), k = 8 * (l / 16) .. + 7:
//     the eight nibbles of payload dword l / 16 of that row's block, spread into bytes by two masks.
//   A operand (16 x 32): the activations, staged as fixed point scaled per block (x = xs * q, xs = the block's largest
//     magnitude / the largest q) and cut into signed byte digits.  Five to eight activation rows: two digits each
//     (q = 256 hi + lo, 16 bits), operand row m = 2 b + digit, so eight rows fill the operand and nothing of the
//     instruction is idle.  Up to four rows ("wide"): three digits each (24 bits), m = 4 b + digit.
//   D (16 x 16): lane l receives column n = l % 16, rows m = 4 (l / 16) .. + 3, i.e. for ITS weight row both digits
//     of activation rows 2 (l / 16) and 2 (l / 16) + 1 (wide: the three digits of row l / 16).  256 hi + lo is one
//     integer multiply-add, and
//       y[b, n] += (scale_n * xs_b) * (256 hi + lo) + bias_n * (xs_b * sum of the block's fixed-point x)
//     needs the block header of the lane's own row only: no value crosses lanes after the instruction, and every
//     lane owns two outputs of its row from the first block to the last.
// Per instruction (16 rows x 32 weights = 320 bytes of weights): 3 operations to spread the nibbles, 2 to convert the
// header, 10 for the two outputs.  Four SIMDs at that rate consume weights several times faster than memory
// delivers them, which the 4x4x4 f16 kernel (eight instructions and their operand shuffles per block of four rows)
// does not.
//
// Memory.  A unit is 16 rows x 8 blocks (2.5 KB).  Lane l loads block l % 8 of rows l / 8 and l / 8 + 8 as whole
// 20-byte blocks (dwordx4 + dword, 160 contiguous bytes per row), keeps four units in flight in registers, and
// passes the blocks through a wave-private LDS tile to reach the operand layout (row pitch 44 dwords: the 16 rows
// x 4 dwords a read touches fall into 64 different banks).  Nothing is fetched twice; no barrier: a wave's LDS
// accesses are carried out in order.
//
// Work split.  A workgroup takes tiles of 16 rows (tile = blockIdx, then += gridDim); its waves split K in chunks
// of 8 blocks and add their partial sums through LDS in wave order.  Each wave stages the activations of its own
// chunks only, once for all tiles of the workgroup, behind its first weight loads.
//
// LoRA.  The factor t = A . x of the adapter (of every view's adapter) is either in memory when the launch starts
// (lora.t / mv.t), or computed by the launch itself (lora.slots set): the first lora.rank workgroups are producers,
// one per row of A (the views' A stacked), each forming that row's dot products with the batch's activation rows
// and publishing them as {value, tag of the launch} words; the other workgroups pick them up into LDS after their
// staging barrier, by which time the producers, who have nothing else to do, are long done.  The launcher adds the
// producers only where CUs are idle anyway (tiles + producers <= CUs): a matrix of 2560 rows occupies 160.  A value
// that has not arrived after the poll limit is computed by the wave that misses it, in the producers' order of
// summation (same bits), and counted in sync[2].
//
// Precision.  The weights enter exactly, the integer sums are exact.  An activation is rounded to a multiple of its
// block's largest magnitude / 32639 (two digits: step 3e-5 of the block maximum, against 5e-4 of the element for the
// f16 rounding of the 4x4x4 kernel and of the reference's tiled kernel, shaders/gemm_q4_tiled.metal:45-48) or
// / 8355711 (wide: 1.2e-7, the resolution of the f32 activation itself, so up to four rows track an f32 GEMV as the
// reference's gemm_q4 does).  Any finite f32 activation is in range (the scale is per block); a block whose largest
// magnitude is below 2^-100 counts as zero; an infinite or NaN activation makes the outputs of its row NaN.
#include "lq4_internal.hpp"

#include <type_traits>

namespace lq4 {

namespace {

typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kBpw = 8;            // blocks per wave chunk
constexpr int kTilePitch = 44;     // dwords per row of the LDS tile (40 used; 44 r mod 64 differs for every r < 16)
constexpr int kTileDwords = 16 * kTilePitch;
constexpr int kXqBytes = 512;      // per block: [4 k groups][16 operand rows] x 8 bytes
constexpr int kXfBytes = 64;       // per block: [4 lane groups][xs of rows 2g, 2g + 1, then their sums] f32

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

// WIDE: up to four activation rows at three digits; else up to eight at two.
// CW x TW waves: CW waves split the chunks of one tile, TW tiles are worked on side by side.
// MULTI: the rows are those of several matrices stacked one under the other (MultiViews: view v = rows [begin[v],
// begin[v + 1]), every view a whole number of 16-row tiles), each with its own output [batch, rows of the view] and its
// own LoRA factors; w, y, y_stride and lora are then unused.
template <int CW, int TW, bool WIDE, bool MULTI>
__global__ __launch_bounds__(64 * CW * TW) void gemv_q4_i8(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                           const float* __restrict__ x, uint32_t x_stride,
                                                           uint32_t batch, float* __restrict__ y, uint32_t y_stride,
                                                           LoraEpilogue lora, MultiViews mv) {
    constexpr int WAVES = CW * TW;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // ---- producers of the LoRA factors (see the head of the file): workgroup p < prod owns stacked row p of A ----
    const uint32_t prod = lora.slots ? lora.rank : 0;  // (several views: lora.rank is the ranks of all views together)
    auto a_row_of = [&](uint32_t p, const void*& a, int& a_is_f16, uint32_t& j) {
        a = lora.a;
        a_is_f16 = lora.b_is_f16;
        j = p;
        if constexpr (MULTI) {
            uint32_t v = 0;
#pragma unroll
            for (int i = 1; i < kMaxViews; ++i) v += (static_cast<uint32_t>(i) < mv.count && p >= mv.t_off[i]) ? 1u : 0u;
            a = mv.a[v];
            a_is_f16 = mv.b_is_f16[v];
            j = p - mv.t_off[v];
        }
    };
    if (blockIdx.x < prod) {
        const void* a;
        int a_is_f16;
        uint32_t j;
        a_row_of(blockIdx.x, a, a_is_f16, j);
        // a wave per activation row: no barrier, nothing through LDS, one cross-lane sum before the word goes out
        for (uint32_t b = wave; b < batch; b += WAVES) {
            const float total = wave_sum(lora_a_row_partial(a, a_is_f16, j, k, x + static_cast<size_t>(b) * x_stride, lane, 64));
            const unsigned long long word = (static_cast<unsigned long long>(launch_tag()) << 32) | as_u32(total);
            if (lane == 0) __hip_atomic_store(&lora.slots[blockIdx.x * 8 + b], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    const uint32_t wg = blockIdx.x - prod, n_wg = gridDim.x - prod;  // this workgroup among those that stream weights
    const uint32_t tw = wave / CW, cw = wave % CW;
    const uint32_t nb = k / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    // LDS: [nb] activation digits | [nb] activation scales and sums | [WAVES] tiles | [WAVES][64][2] partial sums |
    // [8][64] LoRA factors
    uint8_t* const xq = smem;
    uint8_t* const xf = xq + static_cast<size_t>(nb) * kXqBytes;
    uint32_t* const tile = reinterpret_cast<uint32_t*>(xf + static_cast<size_t>(nb) * kXfBytes) + wave * kTileDwords;
    float* const part = reinterpret_cast<float*>(xf + static_cast<size_t>(nb) * kXfBytes) + WAVES * kTileDwords;
    float* const t_lds = part + WAVES * 64 * 2;  // [8 activation rows][kMaxLoraRank]: the factors picked up from the producers

    const uint32_t n_tiles = (n + 15) / 16;
    const uint32_t chunks = (nb + kBpw - 1) / kBpw;
    const uint32_t my_chunks = cw < chunks ? (chunks - cw + CW - 1) / CW : 0;  // chunk c * CW + cw
    // tiles of the workgroup: blockIdx + j * gridDim; of this wave: j = tw, tw + TW, ...; a round = TW tiles
    const uint32_t wg_tiles = wg < n_tiles ? (n_tiles - wg + n_wg - 1) / n_wg : 0;
    const uint32_t rounds = (wg_tiles + TW - 1) / TW;
    const uint32_t my_tiles = tw < wg_tiles ? (wg_tiles - tw + TW - 1) / TW : 0;
    const uint32_t units = my_tiles * my_chunks;  // unit u = (my tile u / my_chunks, my chunk u % my_chunks)
    auto first_row = [&](uint32_t t) { return (wg + (t * TW + tw) * n_wg) * 16; };
    // MULTI: the view that holds stacked row `row` (uniform: called with a tile's first row)
    auto view_of = [&](uint32_t row) {
        uint32_t v = 0;
        if constexpr (MULTI) {
#pragma unroll
            for (int i = 1; i < kMaxViews; ++i) v += (static_cast<uint32_t>(i) < mv.count && row >= mv.begin[i]) ? 1u : 0u;
        }
        return v;
    };

    auto r_of = [](int l) { return static_cast<uint32_t>(l & 15); };  // the weight row of the tile a lane's outputs belong to
    // load mapping: lane = (block jl, row rq), rows rq + kRowStep * i
    constexpr int kRowStep = 64 / kBpw, kLoads = 16 / kRowStep;
    const uint32_t jl = lane % kBpw, rq = lane / kBpw;
    auto load_unit = [&](Q4BlockRaw (&buf)[kLoads], uint32_t u) {
        const uint32_t t = u / my_chunks, c = u - t * my_chunks;
        const uint32_t row0 = first_row(t);
        uint32_t blk = (c * CW + cw) * kBpw + jl;
        if (blk >= nb) blk = nb - 1;
        const uint8_t* wv = w;
        uint32_t row_base = 0, row_end = n;
        if constexpr (MULTI) {
            const uint32_t v = view_of(row0);
            wv = mv.w[v];
            row_base = mv.begin[v];
            row_end = mv.begin[v + 1];
        }
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            uint32_t row = row0 + rq + kRowStep * i;
            if (row >= row_end) row = row_end - 1;
            row -= row_base;
            const uint8_t* bp = wv + row * row_bytes + blk * static_cast<uint32_t>(kBlockBytes);
            // (plain loads: a unit's 160-byte pieces share their cache lines with the neighbouring waves' pieces)
            buf[i].sb = *reinterpret_cast<const uint32_t*>(bp);
            typedef uint32_t u32x4u __attribute__((ext_vector_type(4), aligned(4)));
            const u32x4u q = *reinterpret_cast<const u32x4u*>(bp + 4);
            buf[i].q[0] = q.x; buf[i].q[1] = q.y; buf[i].q[2] = q.z; buf[i].q[3] = q.w;
        }
    };

    // ---- stage the activations, all waves together: task = (block, activation row, k group), 8 values each ----
    // The values of a thread's first tasks are requested before any weight (loads are answered in the order a CU
    // issued them: behind the weight prefetch the staging would wait for the weights), all at once.
    constexpr uint32_t kRows = WIDE ? 4 : 8;      // activation rows the operand holds
    constexpr int kHoist = WAVES >= 16 ? 2 : 4;   // tasks a thread requests ahead (K = 2048 at eight rows: all of them)
    // q = rint(x / xs) with xs = block maximum / kQScale: |q| stays below kQScale + 2 whatever the rounding of the
    // reciprocal, every digit within -128..127; wide: 22 bits and sign, what the float trick below can hold
    constexpr float kQScale = WIDE ? 4194000.0f : 32639.0f;
    const uint32_t n_tasks = nb * 4 * kRows;
    auto task_ptr = [&](uint32_t idx) {
        const uint32_t kg = idx & 3, b = (idx >> 2) & (kRows - 1), blk = idx / (4 * kRows);
        // rows and blocks that do not exist re-read an existing one; their digits are zeroed below
        const uint32_t bb = b < batch ? b : 0, bl = blk < nb ? blk : nb - 1;
        return reinterpret_cast<const float4*>(x + static_cast<size_t>(bb) * x_stride + bl * kBlockWeights + kg * 8);
    };
    auto quad_max = [](uint32_t v) {
        v = max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false)));
        return max(v, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false)));
    };
    auto quad_sum = [](int v) {
        v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);
        return v + __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);
    };
    auto stage_task = [&](uint32_t idx, const float4 xa, const float4 xb) {
        const uint32_t kg = idx & 3, b = (idx >> 2) & (kRows - 1), blk = idx / (4 * kRows);
        const bool live = blk < nb && b < batch;  // (the four lanes of a (block, row) agree)
        const float v[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
        // largest magnitude as a bit pattern: infinities and NaNs come out on top of every finite value
        uint32_t abits = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) abits = max(abits, as_u32(v[i]) & 0x7FFFFFFFu);
        abits = quad_max(live ? abits : 0u);
        const bool finite = abits < 0x7F800000u;
        float inv = 0.0f, xs = 0.0f;
        if (finite && abits >= 0x0D800000u) {  // 2^-100 and up
            xs = as_f32(abits) * (1.0f / kQScale);
            inv = __builtin_amdgcn_rcpf(xs);
        } else if (!finite) {
            xs = as_f32(0x7FC00000u);  // infinite or NaN activation: the row's outputs become NaN
        }
        // 1.5 * 2^23 + q as a float has q in its low 23 bits in two's complement: bits = 0x4B400000 + q
        uint32_t qb[8], sum_bits = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            qb[i] = as_u32(fmaf(v[i], inv, 12582912.0f));  // (a row that does not exist: inv = 0, digits 0)
            sum_bits += qb[i];
        }
        const int sum = quad_sum(static_cast<int>(sum_bits - 8u * 0x4B400000u));
        // Digits -128..127 from the lowest up: byte 0 of q, byte 1 of q + 0x80, byte 2 of q + 0x8080 (minus the
        // 0x40 the float's own bits hold there).  Byte p of an operand word pair = element {0, 2, 4, 6, 1, 3, 5,
        // 7}[p] of the k group: the order in which the two masks lay out a payload dword's nibbles.
        constexpr int kDigits = WIDE ? 3 : 2;
        uint32_t dg[kDigits][2];
#pragma unroll
        for (int t = 0; t < kDigits; ++t) {
            const uint32_t add = t == 0 ? 0u : t == 1 ? 0x80u : 0xFFC08080u;
            // byte t of (qb + add) of four elements into one dword: 0x0c selects a zero byte
            const uint32_t sel_lo = 0x0c0c0400u + 0x0101u * t, sel_hi = 0x04000c0cu + 0x01010000u * t;
#pragma unroll
            for (int h = 0; h < 2; ++h) {  // h = 0: elements 0, 2, 4, 6;  h = 1: elements 1, 3, 5, 7
                const uint32_t e0 = qb[h] + add, e1 = qb[2 + h] + add, e2 = qb[4 + h] + add, e3 = qb[6 + h] + add;
                dg[t][h] = __builtin_amdgcn_perm(e1, e0, sel_lo) | __builtin_amdgcn_perm(e3, e2, sel_hi);
            }
        }
        if (blk < nb) {
            // operand row of (b, digit): the highest digit first
            uint2* dst = reinterpret_cast<uint2*>(xq + static_cast<size_t>(blk) * kXqBytes + kg * 128 + ((WIDE ? 4 : 2) * b) * 8);
#pragma unroll
            for (int t = 0; t < kDigits; ++t) dst[t] = make_uint2(dg[kDigits - 1 - t][0], dg[kDigits - 1 - t][1]);
            if (WIDE) dst[3] = make_uint2(0u, 0u);
            if (kg == 0) {
                // per lane group g of the product: {xs, xs} then {sum, sum} of rows 2g, 2g + 1; wide: {xs, sum} of row g
                float* f = reinterpret_cast<float*>(xf + static_cast<size_t>(blk) * kXfBytes);
                const float sx = xs * static_cast<float>(sum);
                if (WIDE) {
                    f[4 * b] = xs;
                    f[4 * b + 1] = sx;
                } else {
                    f[4 * (b >> 1) + (b & 1)] = xs;
                    f[4 * (b >> 1) + 2 + (b & 1)] = sx;
                }
            }
        }
    };

    // The LoRA factor B of the wave's first tile (its first sixteen ranks, f16 in eights) is requested before
    // anything else and used in that tile's epilogue: requested there, its whole latency stood between the last
    // matrix instruction and the store, and a workgroup of these launches has one tile or two.
    struct alignas(16) H8 { _Float16 v[8]; };
    H8 b_pre[2] = {};
    bool use_pre = false;
    if (cw == 0 && my_tiles) {  // uniform
        const uint32_t row0 = first_row(0);
        const void* bq = lora.b;
        uint32_t rank = lora.rank, row_end = n, row_base = 0;
        int b16 = lora.b_is_f16;
        if constexpr (MULTI) {
            const uint32_t v = view_of(row0);
            bq = mv.b[v];
            rank = mv.rank[v];
            b16 = mv.b_is_f16[v];
            row_end = mv.begin[v + 1];
            row_base = mv.begin[v];
        }
        if (rank && b16 && rank % 8 == 0) {
            use_pre = true;
            const uint32_t row = (row0 + r_of(lane) < row_end ? row0 + r_of(lane) : row_end - 1) - row_base;
            const _Float16* brow = static_cast<const _Float16*>(bq) + static_cast<size_t>(row) * rank;
            b_pre[0] = *reinterpret_cast<const H8*>(brow);
            b_pre[1] = *reinterpret_cast<const H8*>(brow + (rank >= 16 ? 8 : 0));
        }
    }
    float4 xv[kHoist][2];
#pragma unroll
    for (int it = 0; it < kHoist; ++it) {
        const float4* xp = task_ptr(tid + it * 64 * WAVES);
        xv[it][0] = xp[0];
        xv[it][1] = xp[1];
    }
    // kDepth units per wave in registers (beside the one in its LDS tile), in a ring of register buffers that the
    // unrolled loop below walks with compile-time indices.  One: the next unit is on its way while the current one is
    // multiplied.  A ring of four was measured slower on the large matrices (12288 x 2048 at 8 / 4 rows 10.0 / 9.2 ->
    // 9.1 / 8.2 us, 2048 x 6144 11.3 -> 10.5) and level on the small ones, where a wave has one unit anyway: what a
    // CU asks for beyond its share of the memory system queues in front of the activations the staging waits for.
    constexpr int kDepth = 1;
    Q4BlockRaw ring[kDepth][kLoads];
#pragma unroll
    for (int i = 0; i < kDepth; ++i) {
        if (static_cast<uint32_t>(i) < units) load_unit(ring[i], i);
    }
    __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled above these loads
    // The LoRA factors of the producers: item i = (stacked row of A i / 8, activation row i % 8), thread i looks at
    // item i while it still has staging to do (the producers need about 2 us, the activations arrive after 1.5),
    // so that in the usual case the value is there when the staging is, and one barrier publishes both.
    const uint32_t tag = launch_tag();
    const unsigned long long none = static_cast<unsigned long long>(tag) << 32;  // lanes without an item: as if published
    const bool early_mine = static_cast<uint32_t>(tid) < prod * 8 && (static_cast<uint32_t>(tid) & 7) < batch;
    unsigned long long early = none;
#pragma unroll
    for (int it = 0; it < kHoist; ++it) {
        if (it == kHoist - 1 && early_mine && lora.spin_limit)
            early = __hip_atomic_load(&lora.slots[tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t idx = tid + it * 64 * WAVES;
        if (idx < n_tasks) stage_task(idx, xv[it][0], xv[it][1]);  // (whole quads: n_tasks is a multiple of 4)
    }
    for (uint32_t idx = tid + kHoist * 64 * WAVES; idx < n_tasks; idx += 64 * WAVES) {
        const float4* xp = task_ptr(idx);
        stage_task(idx, xp[0], xp[1]);
    }
    if (prod && static_cast<uint32_t>(tid) < prod * 8)
        t_lds[(tid & 7) * kMaxLoraRank + (tid >> 3)] = early_mine ? as_f32(static_cast<uint32_t>(early)) : 0.0f;
    __syncthreads();
    // A wave some of whose values were not there yet (or that has more items than lanes) goes the patient way.  No
    // barrier of its own: whoever reads t_lds does so in a tile's epilogue, behind the two barriers of the partial
    // sums that every wave passes once a round (a workgroup of one wave reads its own writes).
    const bool early_bad = early_mine && (!lora.spin_limit || static_cast<uint32_t>(early >> 32) != tag);
    if (prod && (__any(early_bad) || prod * 8 > 64 * WAVES)) {  // uniform in the wave
        for (uint32_t i0 = wave * 64; i0 < prod * 8; i0 += 64 * WAVES) {  // uniform
            const uint32_t i = i0 + lane;
            const bool mine = i < prod * 8 && (i & 7) < batch;
            // first through the caches (the usual case: the producers are done, one fetch per XCD), then past them
            unsigned long long v = none;
            if (lora.spin_limit) {
                if (mine) v = *static_cast<const volatile unsigned long long*>(&lora.slots[i]);
                for (uint32_t spin = 0; spin < lora.spin_limit && !__all(static_cast<uint32_t>(v >> 32) == tag); ++spin) {
                    __builtin_amdgcn_s_sleep(4);
                    if (mine) v = __hip_atomic_load(&lora.slots[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            } else if (mine) {
                v = 0;  // (no polling at all: every item is computed here)
            }
            float val = as_f32(static_cast<uint32_t>(v));
            uint64_t missing = __ballot(static_cast<uint32_t>(v >> 32) != tag);
            while (missing) {  // uniform: the wave computes the item itself, in the producers' order of summation
                const uint32_t fl = static_cast<uint32_t>(__builtin_ctzll(missing));
                missing &= missing - 1;
                const uint32_t item = i0 + fl;
                const void* a;
                int a_is_f16;
                uint32_t j;
                a_row_of(item >> 3, a, a_is_f16, j);
                const float* xr = x + static_cast<size_t>(item & 7) * x_stride;
                const float total = wave_sum(lora_a_row_partial(a, a_is_f16, j, k, xr, lane, 64));
                if (static_cast<uint32_t>(lane) == fl) val = total;
                if (lane == 0) __hip_atomic_fetch_add(&lora.sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (i < prod * 8) t_lds[(i & 7) * kMaxLoraRank + (i >> 3)] = mine ? val : 0.0f;
        }
    }

    // ---- the product ----
    const uint32_t r = lane & 15, g = lane >> 4;  // operand mapping: weight row r of the tile, k group / row pair g
    float acc0 = 0.0f, acc1 = 0.0f;
    auto process = [&](Q4BlockRaw (&cur)[kLoads], uint32_t u) {
        if (u >= units) return;  // uniform
        // through the tile: tile[row][5 * block + d]; the buffer is then free for the unit kDepth ahead
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            uint32_t* tp = tile + (rq + kRowStep * i) * kTilePitch + 5 * jl;
            tp[0] = cur[i].sb;
            tp[1] = cur[i].q[0]; tp[2] = cur[i].q[1]; tp[3] = cur[i].q[2]; tp[4] = cur[i].q[3];
        }
        if (u + kDepth < units) load_unit(cur, u + kDepth);  // uniform
        const uint32_t t = u / my_chunks, c = u - t * my_chunks;
        const uint32_t blk0 = (c * CW + cw) * kBpw;
        const uint32_t* tr = tile + r * kTilePitch;
        // four blocks at a time, straight-line: their LDS reads, then their four matrix instructions back to back,
        // then their results (a block past the end of the row re-reads the row's last one and counts for nothing)
#pragma unroll
        for (int j0 = 0; j0 < kBpw; j0 += 4) {
            uint32_t sb[4], qd[4];
            long aop[4];
            float4 f[4];
            bool live[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const uint32_t blk_raw = blk0 + j0 + jj;
                live[jj] = blk_raw < nb;  // uniform
                const uint32_t blk = live[jj] ? blk_raw : nb - 1;
                sb[jj] = tr[5 * (j0 + jj)];
                qd[jj] = tr[5 * (j0 + jj) + 1 + g];
                aop[jj] = *reinterpret_cast<const long*>(xq + static_cast<size_t>(blk) * kXqBytes + lane * 8);
                f[jj] = *reinterpret_cast<const float4*>(xf + static_cast<size_t>(blk) * kXfBytes + g * 16);
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
                const float scale = live[jj] ? half_lo(sb[jj]) : 0.0f, bias = live[jj] ? half_hi(sb[jj]) : 0.0f;
                if constexpr (WIDE) {
                    // the top digit's sum times 2^16 is exact in f32, so is 256 mid + low: one rounding in the add
                    const float d0 = fmaf(static_cast<float>(d[jj].x), 65536.0f, static_cast<float>(d[jj].y * 256 + d[jj].z));
                    acc0 = fmaf(scale * f[jj].x, d0, acc0);
                    acc0 = fmaf(bias, f[jj].y, acc0);
                } else {
                    const float d0 = static_cast<float>(d[jj].x * 256 + d[jj].y), d1 = static_cast<float>(d[jj].z * 256 + d[jj].w);
                    acc0 = fmaf(scale * f[jj].x, d0, acc0);
                    acc1 = fmaf(scale * f[jj].y, d1, acc1);
                    acc0 = fmaf(bias, f[jj].z, acc0);
                    acc1 = fmaf(bias, f[jj].w, acc1);
                }
            }
        }
        if (c + 1 == my_chunks) {  // the wave's part of the tile is complete: meet the tile's other waves in LDS
            const uint32_t row = first_row(t) + r;
            if constexpr (WAVES > 1) {
                __syncthreads();  // (every wave passes here once a round; waves without work bring zeros)
                part[(wave * 64 + lane) * 2] = acc0;
                part[(wave * 64 + lane) * 2 + 1] = acc1;
                __syncthreads();
                acc0 = 0.0f;
                acc1 = 0.0f;
                if (cw == 0) {
#pragma unroll
                    for (int v = 0; v < CW; ++v) {
                        acc0 += part[((tw * CW + v) * 64 + lane) * 2];
                        acc1 += part[((tw * CW + v) * 64 + lane) * 2 + 1];
                    }
                }
            }
            if (cw == 0 && row < n) {
                const uint32_t b0 = WIDE ? g : 2 * g, b1 = WIDE ? batch : 2 * g + 1;  // (wide: one row a lane)
                // this row's adapter and output: the launch's, or (several views) those of the tile's view
                LoraEpilogue lo = lora;
                float* yv = y;
                uint32_t ys = y_stride, lrow = row;
                if constexpr (MULTI) {
                    const uint32_t v = view_of(first_row(t));
                    lo.b = mv.b[v];
                    lo.t = mv.t[v];
                    lo.rank = mv.rank[v];
                    lo.b_is_f16 = mv.b_is_f16[v];
                    lo.scale = mv.scale[v];
                    yv = mv.y[v];
                    ys = mv.begin[v + 1] - mv.begin[v];
                    lrow = row - mv.begin[v];
                }
                // t of activation rows b0 and b1, `t0[i]` = factor i: from memory, or (producers) from LDS
                auto delta = [&](auto* t0, auto* t1) {
                    // (every load below is unconditional and used where it is made: a load left pending on one path
                    // would make the compiler wait for the whole weight ring wherever its register is reused)
                    float l0 = 0.0f, l1 = 0.0f;
                    if (lo.b_is_f16 && lo.rank % 8 == 0) {
                        // eight factors a step: one 16-byte load of B[row, i..i+7] (the first two steps of the wave's
                        // first tile: requested at the start of the kernel) and four of t
                        const _Float16* brow = static_cast<const _Float16*>(lo.b) + static_cast<size_t>(lrow) * lo.rank;
                        auto eight = [&](const H8& bq, uint32_t i) {
                            const float4 ta = *reinterpret_cast<const float4*>(t0 + i), tb = *reinterpret_cast<const float4*>(t0 + i + 4);
                            const float4 ua = *reinterpret_cast<const float4*>(t1 + i), ub = *reinterpret_cast<const float4*>(t1 + i + 4);
                            const float tv[8] = {ta.x, ta.y, ta.z, ta.w, tb.x, tb.y, tb.z, tb.w};
                            const float uv[8] = {ua.x, ua.y, ua.z, ua.w, ub.x, ub.y, ub.z, ub.w};
#pragma unroll
                            for (int jj = 0; jj < 8; ++jj) {
                                const float bv = static_cast<float>(bq.v[jj]);
                                l0 = fmaf(bv, tv[jj], l0);
                                l1 = fmaf(bv, uv[jj], l1);
                            }
                        };
                        uint32_t i = 0;
                        if (use_pre && t == 0) {  // uniform
                            eight(b_pre[0], 0);
                            if (lo.rank >= 16) eight(b_pre[1], 8);
                            i = lo.rank >= 16 ? 16 : 8;
                        }
                        for (; i < lo.rank; i += 8) eight(*reinterpret_cast<const H8*>(brow + i), i);
                    } else {
                        for (uint32_t i = 0; i < lo.rank; ++i) {
                            const size_t bi = static_cast<size_t>(lrow) * lo.rank + i;
                            const float bv = lo.b_is_f16 ? static_cast<float>(static_cast<const _Float16*>(lo.b)[bi])
                                                         : static_cast<const float*>(lo.b)[bi];
                            l0 = fmaf(bv, t0[i], l0);
                            l1 = fmaf(bv, t1[i], l1);
                        }
                    }
                    acc0 = fmaf(lo.scale, l0, acc0);
                    acc1 = fmaf(lo.scale, l1, acc1);
                };
                if (lo.rank) {
                    const uint32_t c0 = b0 < batch ? b0 : 0, c1 = b1 < batch ? b1 : 0;
                    if (prod) {
                        uint32_t off = 0;
                        if constexpr (MULTI) off = mv.t_off[view_of(first_row(t))];
                        delta(t_lds + c0 * kMaxLoraRank + off, t_lds + c1 * kMaxLoraRank + off);
                    } else {
                        delta(lo.t + c0 * lo.rank, lo.t + c1 * lo.rank);
                    }
                }
                if (b0 < batch) yv[static_cast<size_t>(b0) * ys + lrow] = acc0;
                if (b1 < batch) yv[static_cast<size_t>(b1) * ys + lrow] = acc1;
            }
            acc0 = 0.0f;
            acc1 = 0.0f;
        }
    };

    for (uint32_t u = 0; u < units; u += kDepth) {
#pragma unroll
        for (int i = 0; i < kDepth; ++i) process(ring[i], u + i);
    }
    // a wave meets the others once a round: those with fewer tiles than rounds (or no chunk at all) make up for it
    if constexpr (WAVES > 1) {
        const uint32_t met = my_chunks ? my_tiles : 0;
        for (uint32_t t = met; t < rounds; ++t) {
            __syncthreads();
            part[(wave * 64 + lane) * 2] = 0.0f;
            part[(wave * 64 + lane) * 2 + 1] = 0.0f;
            __syncthreads();
        }
    }
}

struct I8Plan {
    uint32_t cw, tw, grid;
    size_t lds;
};

size_t lds_eight_waves(uint32_t nb) {
    return static_cast<size_t>(nb) * (kXqBytes + kXfBytes) + 8 * kTileDwords * 4 + 8 * 64 * 2 * 4 + 8 * kMaxLoraRank * 4;
}

}  // namespace

// At least two 16-row tiles per CU and rows short enough that two eight-wave workgroups share a CU's LDS.
bool gemv_i8_many_short_rows(uint32_t n, uint32_t k, uint32_t cu_count) {
    const uint32_t nb = k / kBlockWeights;
    return (n + 15) / 16 >= 2 * cu_count && nb >= 4 * kBpw && lds_eight_waves(nb) <= 78 * 1024;
}

namespace {

bool plan_i8(uint32_t n, uint32_t k, uint32_t batch, uint32_t cu_count, I8Plan* out) {
    if (k == 0 || k % kBlockWeights || n == 0 || batch == 0 || batch > 8) return false;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t chunks = (nb + kBpw - 1) / kBpw;
    const uint32_t n_tiles = (n + 15) / 16;
    I8Plan p;
    // waves that split one tile's chunks: a power of two up to sixteen; tiles side by side: as many as fill a
    // sixteen-wave workgroup, but no more than leaves every CU a workgroup (one workgroup a CU stages the
    // activations once for all the tiles that CU works on)
    p.cw = chunks >= 16 ? 16 : chunks >= 8 ? 8 : chunks >= 4 ? 4 : chunks >= 2 ? 2 : 1;
    p.tw = 16 / p.cw;
    while (p.tw > 1 && (n_tiles + p.tw - 1) / p.tw < cu_count) p.tw /= 2;
    for (;;) {
        const uint32_t waves = p.cw * p.tw;
        p.lds = static_cast<size_t>(nb) * (kXqBytes + kXfBytes) + static_cast<size_t>(waves) * kTileDwords * 4 +
                static_cast<size_t>(waves) * 64 * 2 * 4 + 8 * kMaxLoraRank * 4;
        if (p.lds <= 160 * 1024) break;
        if (p.tw > 1) p.tw /= 2;
        else if (p.cw > 1) p.cw /= 2;
        else return false;
    }
    // Many tiles of short rows (12288 x 2048: 768 tiles): workgroups of eight waves (two split K, four tiles side by
    // side), two of which fit a CU, one round each, instead of sixteen-wave workgroups that walk two rounds
    // (at 8 / 4 rows 9.1 / 8.1 -> 8.8 / 7.9 us).
    if (gemv_i8_many_short_rows(n, k, cu_count)) {
        p.cw = 2;
        p.tw = 4;
        p.lds = lds_eight_waves(nb);
        p.grid = (n_tiles + 3) / 4;
        *out = p;
        return true;
    }
    const uint32_t groups = (n_tiles + p.tw - 1) / p.tw;  // rounds of tiles in all
    if (groups <= cu_count) {
        p.grid = groups;
    } else {
        const uint32_t per = (groups + cu_count - 1) / cu_count;
        p.grid = (groups + per - 1) / per;  // the same number of rounds for every workgroup, to within one
    }
    *out = p;
    return true;
}

template <int CW, int TW, bool WIDE, bool MULTI>
void launch_i8(const I8Plan& p, const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride,
               uint32_t batch, float* y, uint32_t y_stride, const LoraEpilogue& lora, const MultiViews& mv,
               hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q4_i8<CW, TW, WIDE, MULTI>), 160 * 1024);
    const uint32_t producers = lora.slots ? lora.rank : 0;
    hipLaunchKernelGGL((gemv_q4_i8<CW, TW, WIDE, MULTI>), dim3(producers + p.grid), dim3(64 * CW * TW), p.lds, stream, w, n,
                       k, x, x_stride, batch, y, y_stride, lora, mv);
}

template <bool WIDE, bool MULTI>
void launch_i8_shape(const I8Plan& p, const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride,
                     uint32_t batch, float* y, uint32_t y_stride, const LoraEpilogue& lora, const MultiViews& mv,
                     hipStream_t stream) {
#define LQ4_I8(CW_, TW_)                \
    if (p.cw == CW_ && p.tw == TW_)     \
    return launch_i8<CW_, TW_, WIDE, MULTI>(p, w, n, k, x, x_stride, batch, y, y_stride, lora, mv, stream)
    LQ4_I8(16, 1);
    LQ4_I8(8, 2); LQ4_I8(8, 1);
    LQ4_I8(4, 4); LQ4_I8(4, 2); LQ4_I8(4, 1);
    LQ4_I8(2, 8); LQ4_I8(2, 4); LQ4_I8(2, 2); LQ4_I8(2, 1);
    LQ4_I8(1, 16); LQ4_I8(1, 8); LQ4_I8(1, 4); LQ4_I8(1, 2); LQ4_I8(1, 1);
#undef LQ4_I8
}

}  // namespace

bool gemv_i8_serves(uint32_t n, uint32_t k, uint32_t batch, uint32_t cu_count) {
    I8Plan p;
    return plan_i8(n, k, batch, cu_count, &p);
}

void launch_gemv_i8(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride, uint32_t batch,
                    float* y, uint32_t y_stride, const LoraEpilogue& lora, uint32_t cu_count, hipStream_t stream) {
    I8Plan p;
    if (!plan_i8(n, k, batch, cu_count, &p)) return;  // the caller asked gemv_i8_serves first
    const MultiViews none{};
    if (batch <= 4) launch_i8_shape<true, false>(p, w, n, k, x, x_stride, batch, y, y_stride, lora, none, stream);
    else launch_i8_shape<false, false>(p, w, n, k, x, x_stride, batch, y, y_stride, lora, none, stream);
}

// The launch can carry `rank_total` producer workgroups for the LoRA factors when they find idle CUs beside the
// workgroups that stream weights (one workgroup runs per CU), the slots (rank_total x 8) and the LDS hold them, and a
// 16-byte row of A can be loaded (K a multiple of 8 elements is given: K is a multiple of 32).
bool gemv_i8_lora_in_launch(uint32_t n, uint32_t k, uint32_t batch, uint32_t rank_total, uint32_t cu_count) {
    I8Plan p;
    return rank_total != 0 && rank_total <= static_cast<uint32_t>(kMaxLoraRank) && plan_i8(n, k, batch, cu_count, &p) &&
           p.grid + rank_total <= cu_count;
}

// The stacked launch serves views that are whole numbers of 16-row tiles.
bool gemv_i8_multi_serves(const MultiViews& mv, uint32_t k, uint32_t batch, uint32_t cu_count) {
    if (mv.count == 0 || mv.count > static_cast<uint32_t>(kMaxViews)) return false;
    for (uint32_t v = 0; v < mv.count; ++v)
        if ((mv.begin[v + 1] - mv.begin[v]) % 16) return false;
    I8Plan p;
    return plan_i8(mv.begin[mv.count], k, batch, cu_count, &p);
}

void launch_gemv_i8_multi(const MultiViews& mv, uint32_t k, const float* x, uint32_t x_stride, uint32_t batch,
                          uint32_t cu_count, const LoraEpilogue* in_launch, hipStream_t stream) {
    const uint32_t n = mv.begin[mv.count];
    I8Plan p;
    if (!plan_i8(n, k, batch, cu_count, &p)) return;  // the caller asked gemv_i8_multi_serves first
    const LoraEpilogue hand = in_launch ? *in_launch : LoraEpilogue{};  // rank = the views' ranks together, slots, sync
    if (batch <= 4) launch_i8_shape<true, true>(p, nullptr, n, k, x, x_stride, batch, nullptr, 0, hand, mv, stream);
    else launch_i8_shape<false, true>(p, nullptr, n, k, x, x_stride, batch, nullptr, 0, hand, mv, stream);
}

}  // namespace lq4
