// Grouped expert GEMV of the MoE path on the matrix cores.
//
// One workgroup handles one expert, one chunk of that expert's output rows and up to four of
// the (token, slot) pairs routed to it; experts nobody chose exit at once.  The expert's Q4
// blocks stream through registers exactly like the small-batch decode GEMV
// (lq4_gemv_mfma.hip): lane 4g+j owns block 16*s + g of weight row 4t + j, a masked dword of
// nibbles is fed to v_mfma_f32_4x4x4_16B_f16 as a pair of f16 subnormals, and every f32
// activation is split x = hi + lo/2048 into two f16 columns, so results track an f32 GEMV.
//
// GATE_UP = true: the two weight rows a lane owns per unit are gate row i and up row I + i of
// the expert ([E, 2I, H], gate rows first: crates/inference/src/model/qwen35/moe.rs:127-190),
// and the workgroup's final phase writes h[pair, i] = silu(g) * u.  GATE_UP = false: plain rows
// of the down projection ([E, H, I]), o[pair, r] = W . h[pair].
#include "lq4_internal.hpp"

#ifndef LQ4_MOE_RING
#define LQ4_MOE_RING 3
#endif

namespace lq4 {

namespace {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kTok = 4;           // pairs per workgroup pass
constexpr int kCols = 2 * kTok;   // hi and lo column per pair
constexpr float kLoScale = 2048.0f;
constexpr float kTwo24 = 16777216.0f;
constexpr int kRing = LQ4_MOE_RING;
constexpr uint32_t kPitch16 = (kCols * 64 + 16) / 16;  // per K block: 8 columns of 32 f16, then 4 sums

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;
    uint32_t q[4];
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

__device__ __forceinline__ float silu(float v) { return v * (1.0f / (1.0f + expf(-v))); }

struct MoeGemvArgs {
    const uint8_t* w;        // expert-major Q4 tensor
    const float* x;          // activation rows
    float* out;              // h (GATE_UP) or o
    const int32_t* offsets;  // [E + 1]
    const int32_t* order;    // pair indices grouped by expert
    const int32_t* ids;      // routed expert of every pair; not null = find the expert's pairs here
    uint32_t n_pairs;        // instead of in offsets/order (few pairs: saves a launch and two dependent loads)
    uint32_t rows_per_expert;  // weight rows of one expert (2I or H)
    uint32_t out_rows;         // output rows per pair (I or H)
    uint32_t k;                // reduction length (H or I)
    uint32_t x_stride;         // floats between activation rows
    uint32_t x_div;            // activation row of a pair = pair / x_div (top_k for x, 1 for h)
    uint32_t tp_per_wave;      // tile pairs (2 x 4 weight rows) per wave
    const uint8_t* w_last;     // not null: the last expert of the grid lives here, not behind the others in w
};

// KS: slices of K per workgroup (waves splitting the 16-block steps of a row).
template <bool GATE_UP, int KS>
__global__ __launch_bounds__(kThreads) void moe_expert_mfma(MoeGemvArgs p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr int RS = 4 / KS;
    // (expert, pass) of this workgroup.  An expert with tensors of its own (w_last) is one that every token
    // chose: all its passes are full-length work, so they are dispatched first instead of forming the tail
    // of the launch (the grid is walked x, then y, then z).
    uint32_t e = blockIdx.y, pass = blockIdx.z;
    if (p.w_last != nullptr) {
        const uint32_t lin = blockIdx.z * gridDim.y + blockIdx.y;
        if (lin < gridDim.z) {
            e = gridDim.y - 1;
            pass = lin;
        } else {
            pass = (lin - gridDim.z) / (gridDim.y - 1);
            e = (lin - gridDim.z) - pass * (gridDim.y - 1);
        }
    }
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __shared__ int32_t s_pair[kTok];  // the pairs of this pass, ascending pair index (= the stable grouping order)
    __shared__ int32_t s_cnt[kThreads / 64];
    int nt;  // pairs in this pass
    if (p.ids) {
        // Every workgroup scans the routing table itself: rank of a matching pair = matches before it.
        const int first = static_cast<int>(pass) * kTok;
        int base = 0;
        for (uint32_t c0 = 0; c0 < p.n_pairs; c0 += kThreads) {
            const uint32_t pi = c0 + tid;
            const bool hit = pi < p.n_pairs && p.ids[pi] == static_cast<int32_t>(e);
            const uint64_t mask = __ballot(hit);
            if (lane == 0) s_cnt[wave] = __popcll(mask);
            __syncthreads();
            int before = base;
            for (int w2 = 0; w2 < wave; ++w2) before += s_cnt[w2];
            const int rank = before + __popcll(mask & ((1ull << lane) - 1ull));
            if (hit && rank >= first && rank < first + kTok) s_pair[rank - first] = static_cast<int32_t>(pi);
            base += s_cnt[0] + s_cnt[1] + s_cnt[2] + s_cnt[3];
            __syncthreads();
        }
        if (base <= first) return;
        nt = base - first < kTok ? base - first : kTok;
    } else {
        const int32_t beg = p.offsets[e] + static_cast<int32_t>(pass) * kTok;
        const int32_t end = p.offsets[e + 1];
        if (beg >= end) return;
        nt = end - beg < kTok ? end - beg : kTok;
        if (tid < nt) s_pair[tid] = p.order[beg + tid];
        __syncthreads();
    }
    const int g = lane >> 2, j = lane & 3;
    const int ks = wave % KS, rs = wave / KS;
    const uint32_t nb = p.k / kBlockWeights;
    const uint32_t nsteps = (nb + 15) / 16;
    const uint32_t n_local = static_cast<uint32_t>(ks) < nsteps ? (nsteps - ks + KS - 1) / KS : 0;
    const uint32_t tp = p.tp_per_wave;
    const uint32_t units = tp * n_local;
    // output rows: a tile pair is 4 (GATE_UP) or 8 (down) of them
    constexpr uint32_t kRowsPerTp = GATE_UP ? 4 : 8;
    const uint32_t rows_per_wg = RS * tp * kRowsPerTp;
    const uint32_t row0 = blockIdx.x * rows_per_wg + rs * tp * kRowsPerTp;

    uint4* const xs16 = reinterpret_cast<uint4*>(smem);
    uint4* const zero_region = xs16 + nb * kPitch16;  // 64 B of zeros
    float* const red = reinterpret_cast<float*>(zero_region + 4);  // [4 waves][tp][2][kCols][4]

    const uint32_t* wbase = (p.w_last != nullptr && e == gridDim.y - 1)
                                ? reinterpret_cast<const uint32_t*>(p.w_last)
                                : reinterpret_cast<const uint32_t*>(p.w) +
                                      static_cast<size_t>(e) * p.rows_per_expert * (nb * 5);

    auto load_unit = [&](Q4BlockRaw (&buf)[2], uint32_t u) {
        const uint32_t t = n_local ? u / n_local : 0, q = u - t * n_local;
        uint32_t blk = (ks + q * KS) * 16 + g;
        if (blk >= nb) blk = nb - 1;
        uint32_t ra = row0 + t * kRowsPerTp + j;
        if (ra >= p.out_rows) ra = p.out_rows - 1;
        uint32_t rb = GATE_UP ? p.out_rows + ra : ra + 4;
        if (!GATE_UP && rb >= p.out_rows) rb = p.out_rows - 1;
        buf[0] = *reinterpret_cast<const Q4BlockRaw*>(wbase + static_cast<size_t>(ra) * (nb * 5) + blk * 5);
        buf[1] = *reinterpret_cast<const Q4BlockRaw*>(wbase + static_cast<size_t>(rb) * (nb * 5) + blk * 5);
    };

    // ---- stage the activations of this pass: 8 values per (block, dword) item per pair ---------
    // All (pair, item) combinations of the pass are flattened and taken four at a time, so the loads
    // of different pairs are in flight together.
    const uint32_t items = nb * 4;
    const float* xrow[kTok];
#pragma unroll
    for (int b = 0; b < kTok; ++b) {
        const int32_t pair = s_pair[b < nt ? b : 0];
        xrow[b] = p.x + static_cast<size_t>(static_cast<uint32_t>(pair) / p.x_div) * p.x_stride;
    }
    constexpr int G = 4;
    const uint32_t total = static_cast<uint32_t>(nt) * items;
    // (a pass with few items leaves slots of the round empty: they are skipped, not converted and dropped)
    const int live_slots = total >= G * kThreads ? G : static_cast<int>((total + kThreads - 1) / kThreads);
    struct Round {
        float4 va[G], vb[G];
        uint32_t wb[G], wi[G];
    };
    auto load_round = [&](Round& r, uint32_t w0) {
#pragma unroll
        for (int i = 0; i < G; ++i) {
            if (i >= live_slots) break;  // uniform
            const uint32_t w = w0 + i * kThreads;
            const uint32_t wc = w < total ? w : 0;
            r.wb[i] = wc / items;
            r.wi[i] = wc - r.wb[i] * items;
            const float* xr = r.wb[i] == 0 ? xrow[0] : r.wb[i] == 1 ? xrow[1] : r.wb[i] == 2 ? xrow[2] : xrow[3];
            const float4* xp = reinterpret_cast<const float4*>(xr + (r.wi[i] >> 2) * kBlockWeights + (r.wi[i] & 3) * 8);
            r.va[i] = xp[0];
            r.vb[i] = xp[1];
        }
    };
    auto store_round = [&](const Round& r, uint32_t w0) {
#pragma unroll
        for (int i = 0; i < G; ++i) {
            if (i >= live_slots) break;  // uniform
            const uint32_t blk = r.wi[i] >> 2, dw = r.wi[i] & 3, bb = r.wb[i];
            const float v[8] = {r.va[i].x, r.va[i].y, r.va[i].z, r.va[i].w, r.vb[i].x, r.vb[i].y, r.vb[i].z, r.vb[i].w};
            _Float16 h[8], l[8];
#pragma unroll
            for (int e2 = 0; e2 < 8; ++e2) {
                const float sc = (e2 & 1) ? v[e2] * 0.0625f : v[e2];
                h[e2] = static_cast<_Float16>(sc);
                l[e2] = static_cast<_Float16>((sc - static_cast<float>(h[e2])) * kLoScale);
            }
            uint4 hi, lo;
            hi.x = pack_h2(h[0], h[4]); hi.y = pack_h2(h[1], h[5]); hi.z = pack_h2(h[2], h[6]); hi.w = pack_h2(h[3], h[7]);
            lo.x = pack_h2(l[0], l[4]); lo.y = pack_h2(l[1], l[5]); lo.z = pack_h2(l[2], l[6]); lo.w = pack_h2(l[3], l[7]);
            float sx = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
            sx = dpp_add<0xB1>(sx);  // the 4 items of a block sit in 4 adjacent lanes
            sx = dpp_add<0x4E>(sx);
            if (w0 + i * kThreads < total) {
                uint4* base = xs16 + blk * kPitch16;
                base[(2 * bb) * 4 + dw] = hi;
                base[(2 * bb + 1) * 4 + dw] = lo;
                if (dw == 0) reinterpret_cast<float*>(base + kCols * 4)[bb] = sx;
            }
        }
    };
    // The first round of activations is requested before any weight (clamped, no branch): loads return
    // in order, so behind the weight prefetch its staging and the barrier after it would wait until
    // the first weights have crossed from HBM.
    Round first;
    load_round(first, tid);

    // ring of kRing unit buffers: kRing - 1 units are in flight while one is consumed
    Q4BlockRaw buf[kRing][2];
#pragma unroll
    for (int i = 0; i < kRing - 1; ++i)  // (a wave with fewer units re-reads its last one)
        load_unit(buf[i], static_cast<uint32_t>(i) < units ? i : (units ? units - 1 : 0));
    __builtin_amdgcn_sched_barrier(0);

    store_round(first, tid);
    for (uint32_t w0 = tid + G * kThreads; w0 < total; w0 += G * kThreads) {
        Round r;
        load_round(r, w0);
        store_round(r, w0);
    }
    if (tid < 4) zero_region[tid] = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();

    const int ncols = 2 * nt;
    float acc[2][kCols];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[t][c] = 0.0f;

    auto process = [&](Q4BlockRaw (&cur)[2], Q4BlockRaw (&nxt)[2], uint32_t u) {
        if (u + kRing - 1 < units) load_unit(nxt, u + kRing - 1);
        const uint32_t t_idx = u / n_local, q = u - t_idx * n_local;
        const uint32_t blk_raw = (ks + q * KS) * 16 + g;
        const bool live = blk_raw < nb;
        const uint32_t blk = live ? blk_raw : nb - 1;
        const uint4* xb = xs16 + blk * kPitch16;

        uint32_t a_op[2][16];
#pragma unroll
        for (int set = 0; set < 2; ++set) {
            const int col = 4 * set + j;
            const uint4* src = col < ncols ? xb + col * 4 : zero_region;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 v = src[i];
                a_op[set][4 * i + 0] = v.x; a_op[set][4 * i + 1] = v.y;
                a_op[set][4 * i + 2] = v.z; a_op[set][4 * i + 3] = v.w;
            }
        }
        // sum of a pair's activations over the block (the bias term; it rides on the hi column only)
        const float4 sums = *reinterpret_cast<const float4*>(xb + kCols * 4);
        float sum_x[kTok] = {sums.x, sums.y, sums.z, sums.w};
#pragma unroll
        for (int b = 0; b < kTok; ++b)
            if (b >= nt || !live) sum_x[b] = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            float4v prod[2] = {float4v{0.0f, 0.0f, 0.0f, 0.0f}, float4v{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
            for (int dw = 0; dw < 4; ++dw) {
                const uint32_t qd = cur[t].q[dw];
                const uint32_t q8 = qd >> 8;
                const uint32_t w0 = qd & 0x000F000Fu, w1 = qd & 0x00F000F0u;
                const uint32_t w2 = q8 & 0x000F000Fu, w3 = q8 & 0x00F000F0u;
                const half4 b01 = __builtin_bit_cast(half4, uint2{w0, w1});
                const half4 b23 = __builtin_bit_cast(half4, uint2{w2, w3});
#pragma unroll
                for (int set = 0; set < 2; ++set) {
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
            for (int c = 0; c < kCols; ++c) {
                const float with_bias = (c & 1) ? acc[t][c] : fmaf(bias, sum_x[c / 2], acc[t][c]);
                acc[t][c] = fmaf(d, prod[c / 4][c % 4], with_bias);
            }
        }
    };

    // tile pair finished for this wave: sum over the 16 blocks of a step (lanes with equal j).  A pair's hi
    // and lo column are joined first and only the pairs of this pass are reduced: with short rows (one
    // step per tile pair) the cross-lane sums are a third of the kernel's vector instructions otherwise.
    auto finish = [&](uint32_t t_idx) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int b = 0; b < kTok; ++b) {
                float v = fmaf(acc[t][2 * b + 1], 1.0f / kLoScale, acc[t][2 * b]);
                acc[t][2 * b] = 0.0f;
                acc[t][2 * b + 1] = 0.0f;
                if (b < nt) {  // the same for the whole workgroup
                    v = dpp_add<0x124>(v);  // row_ror:4
                    v = dpp_add<0x128>(v);  // row_ror:8
                    v = sum_over_rows(v);
                    if (lane < 4) red[(((wave * tp + t_idx) * 2 + t) * kTok + b) * 4 + lane] = v;
                }
            }
    };

    if (units) {
        uint32_t q = 0, t_idx = 0;
        for (uint32_t u0 = 0; u0 < units; u0 += kRing) {
#pragma unroll
            for (int i = 0; i < kRing; ++i) {
                if (u0 + i >= units) break;
                process(buf[i], buf[(i + kRing - 1) % kRing], u0 + i);  // refills the buffer consumed last
                if (++q == n_local) { finish(t_idx++); q = 0; }
            }
        }
    } else {
        for (uint32_t t_idx = 0; t_idx < tp; ++t_idx) finish(t_idx);  // zeros: this wave has no K slice
    }
    __syncthreads();

    // ---- final phase: one thread per (output row, pair) -------------------------------------------
    const uint32_t n_out = rows_per_wg * kTok;
    for (uint32_t o = tid; o < n_out; o += kThreads) {
        const uint32_t b = o % kTok, lr = o / kTok;          // pair slot, local output row
        const uint32_t rs_o = lr / (tp * kRowsPerTp);
        const uint32_t in_rs = lr % (tp * kRowsPerTp);
        const uint32_t t_idx = in_rs / kRowsPerTp, in_tp = in_rs % kRowsPerTp;
        const uint32_t jj = in_tp & 3, half = in_tp >> 2;    // half: second tile of a down pair
        const uint32_t row = blockIdx.x * rows_per_wg + lr;
        if (static_cast<int>(b) >= nt || row >= p.out_rows) continue;
        float v[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            float sum = 0.0f;
            for (int s = 0; s < KS; ++s) {
                const uint32_t wv = rs_o * KS + s;
                sum += red[((((wv * tp + t_idx) * 2 + t) * kTok) + b) * 4 + jj];
            }
            v[t] = sum;
        }
        const int32_t pair = s_pair[b];
        p.out[static_cast<size_t>(pair) * p.out_rows + row] = GATE_UP ? silu(v[0]) * v[1] : v[half];
    }
}

template <bool GATE_UP, int KS>
void launch_ks(const MoeGemvArgs& a, uint32_t num_experts, uint32_t max_pairs_per_expert, hipStream_t stream) {
    constexpr uint32_t rows_per_tp = GATE_UP ? 4 : 8;
    const uint32_t rows_per_wg = (4 / KS) * a.tp_per_wave * rows_per_tp;
    const uint32_t nb = a.k / kBlockWeights;
    const size_t lds = static_cast<size_t>(nb) * kPitch16 * 16 + 64 + 4 * a.tp_per_wave * 2 * kCols * 4 * sizeof(float);
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(moe_expert_mfma<GATE_UP, KS>), 159 * 1024);  // the rest is static
    const dim3 grid((a.out_rows + rows_per_wg - 1) / rows_per_wg, num_experts, (max_pairs_per_expert + kTok - 1) / kTok);
    hipLaunchKernelGGL((moe_expert_mfma<GATE_UP, KS>), grid, dim3(kThreads), lds, stream, a);
}

template <bool GATE_UP>
void launch_phase(MoeGemvArgs a, uint32_t num_experts, uint32_t max_pairs_per_expert, hipStream_t stream) {
    const uint32_t nsteps = (a.k / kBlockWeights + 15) / 16;
    constexpr uint32_t rows_per_tp = GATE_UP ? 4 : 8;
    // about 32 (gate/up) or 128 (down) output rows per workgroup: 40-80 KB of blocks each
    // (half of that for a single token's worth of pairs: with so few workgroups at work the chip is
    // filled by more, smaller ones; measured 26.7 -> 23.7 us at 8 pairs, but slower from 128 pairs on)
    const bool few_pairs = a.n_pairs <= 16;
    const uint32_t target_rows = GATE_UP ? (few_pairs ? 16 : 32) : (few_pairs ? 64 : 128);
    // Waves split the output rows; they split K as well only when an expert has too few rows to
    // give every wave a tile pair (each K slice costs a cross-lane reduction per tile pair).
    uint32_t ks = 1;
    while (ks < 4 && ks * 2 <= nsteps && a.out_rows < (4 / ks) * rows_per_tp * 4) ks *= 2;
    a.tp_per_wave = target_rows / ((4 / ks) * rows_per_tp);
    if (a.tp_per_wave < 1) a.tp_per_wave = 1;
    if (ks == 4) launch_ks<GATE_UP, 4>(a, num_experts, max_pairs_per_expert, stream);
    else if (ks == 2) launch_ks<GATE_UP, 2>(a, num_experts, max_pairs_per_expert, stream);
    else launch_ks<GATE_UP, 1>(a, num_experts, max_pairs_per_expert, stream);
}

}  // namespace

size_t moe_mfma_lds_bytes(uint32_t k) {
    return static_cast<size_t>(k / kBlockWeights) * kPitch16 * 16 + 64 + 4 * 8 * 2 * kCols * 4 * sizeof(float);
}

void launch_moe_gate_up_mfma(const uint8_t* gate_up, uint32_t num_experts, uint32_t inter, uint32_t hidden,
                             const float* x, uint32_t tokens, uint32_t top_k, const int32_t* offsets,
                             const int32_t* order, const int32_t* ids, float* h, hipStream_t stream,
                             const uint8_t* last_expert) {
    MoeGemvArgs a{gate_up, x, h, offsets, order, ids, tokens * top_k, 2 * inter, inter, hidden, hidden, top_k, 0,
                  last_expert};
    launch_phase<true>(a, num_experts, tokens, stream);
}

void launch_moe_down_mfma(const uint8_t* down, uint32_t num_experts, uint32_t inter, uint32_t hidden,
                          const float* h, uint32_t tokens, uint32_t top_k, const int32_t* offsets,
                          const int32_t* order, const int32_t* ids, float* o, hipStream_t stream,
                          const uint8_t* last_expert) {
    MoeGemvArgs a{down, h, o, offsets, order, ids, tokens * top_k, hidden, hidden, inter, inter, 1, 0, last_expert};
    launch_phase<false>(a, num_experts, tokens, stream);
}

}  // namespace lq4
