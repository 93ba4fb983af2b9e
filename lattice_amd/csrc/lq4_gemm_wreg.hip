// Prefill GEMM, weights-in-registers variant: Y[M,N] = X[M,K] . W[N,K]^T for large shapes.
//
// A workgroup of four waves owns 128 tokens x 256 weight rows; wave w owns weight rows
// 64w .. 64w+63 against all 128 tokens.  Only the activations go through LDS (f16, double
// buffered, one barrier per 128-wide K step).  Weights never touch LDS: every lane loads whole
// Q4 blocks straight from global memory, dequantises them in registers and feeds them to
// v_mfma_f32_16x16x32_f16 as the A operand.  Compared with staging dequantised weights in LDS
// this removes 2 bytes of LDS write and 2 x 2 bytes of LDS read per weight, and each weight is
// dequantised exactly once per 128 tokens.
//
// The K dimension inside one matrix-core instruction is a sum, so its order is free as long as
// both operands agree.  A K step covers four Q4 blocks; lane (r = lane % 16, g = lane / 16)
// owns block g of weight row r.  Instruction j (0..3) of the step takes dword j of the lane's
// own block: across the four lane groups it covers weights 8j..8j+7 of four different blocks.
// So a lane only ever touches its own block and its own scale and bias.  The activation
// operand is read from LDS at the matching K offset 32g + 8j.  Within a dword the nibble
// pairs come out of the dequantiser as (w0,w4)(w1,w5)(w2,w6)(w3,w7); instead of shuffling
// every weight back into order, the activations are stored to LDS in that same order once.
//
// Dequantised value: half(q*d + b) with one rounding, the rounding point of the reference's
// tiled kernel (shaders/gemm_q4_tiled.metal:57-66); products accumulate in f32.
//
// Weight loads run two K steps ahead of their use (three rotating register sets), activation
// loads one step ahead; the K loop is unrolled by three so that every register set has a fixed
// role at every position.  Out-of-range rows are clamped to valid rows (their results are never
// stored); blocks past the end of K are clamped to valid blocks and given a zero scale and
// bias, so the loop body is free of divergent branches.
#include "lq4_internal.hpp"

#include <type_traits>
#include <utility>

namespace lq4 {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

constexpr int TM = 128;                    // tokens per workgroup
constexpr int TN = 256;                    // weight rows per workgroup
constexpr int TK = 128;                    // K per step: four Q4 blocks
constexpr int kPitch16 = TK * 2 / 16 + 1;  // LDS row pitch in 16-byte units (272 bytes)
constexpr int kBuf16 = TM * kPitch16;      // one activation buffer, in 16-byte units
constexpr int kGroupM = 16;                // token tiles per rasterisation group
constexpr int NU = 4;                      // 16-row weight tiles per wave
constexpr int NT = TM / 16;                // 16-token tiles per workgroup

struct __attribute__((packed, aligned(4))) Q4BlockRaw {
    uint32_t sb;    // f16 scale | f16 bias << 16
    uint32_t q[4];  // 32 nibbles, nibble i of dword j = weight 8j + i
};

// Sibling formats (FMT 1 = Q8_0, 2 = Q3).
struct __attribute__((packed, aligned(2))) Q8BlockRaw {
    uint16_t d;     // f16 scale
    uint32_t q[8];  // 32 x i8, weight i in byte i
};
struct __attribute__((packed, aligned(4))) Q3BlockRaw {
    uint32_t sb;     // f16 scale | f16 bias << 16
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

struct U4 {
    uint32_t v[4];
};

// Dequantisation of one packed dword (weights 8j..8j+7) into f16 weights in the order
// w0 w4 w1 w5 w2 w6 w3 w7, cut into 13 single-instruction steps so that the K loop can place
// them one by one in the shadow of matrix-core instructions.  A masked dword OR-ed into the
// mantissa of 1024.0 (or 64.0) is the pair (1024+n_lo, 1024+n_hi); one packed subtract makes it
// (n_lo, n_hi) exactly, one packed fma applies scale and bias with a single rounding.
struct DqTmp {
    uint32_t q8;   // Q4: dword >> 8;  Q8_0: second sign-flipped dword;  Q3: spread high-plane bits
    uint32_t qa;   // Q8_0: first sign-flipped dword;  Q3: shifted low-plane dword
    half2v t[4];
};
template <int FMT>
struct DqOps {
    static constexpr int kOps = 13;
};
template <>
struct DqOps<1> {
    static constexpr int kOps = 14;
};
template <>
struct DqOps<2> {
    static constexpr int kOps = 24;
};

__device__ __forceinline__ void dq_op_q4(int op, uint32_t q, half2v d2, half2v b2, DqTmp& tmp, U4& out) {
    const half2v k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
    const half2v k64 = {static_cast<_Float16>(64.0f), static_cast<_Float16>(64.0f)};
    switch (op) {
        case 0: tmp.q8 = q >> 8; break;
        case 1: tmp.t[0] = as_h2(and_or(q, 0x000F000Fu, 0x64006400u)); break;
        case 2: tmp.t[1] = as_h2(and_or(q, 0x00F000F0u, 0x54005400u)); break;
        case 3: tmp.t[2] = as_h2(and_or(tmp.q8, 0x000F000Fu, 0x64006400u)); break;
        case 4: tmp.t[3] = as_h2(and_or(tmp.q8, 0x00F000F0u, 0x54005400u)); break;
        case 5: tmp.t[0] -= k1024; break;
        case 6: tmp.t[1] -= k64; break;
        case 7: tmp.t[2] -= k1024; break;
        case 8: tmp.t[3] -= k64; break;
        default: out.v[op - 9] = as_u32(__builtin_elementwise_fma(tmp.t[op - 9], d2, b2)); break;
    }
}

// Q8_0, weights 8j..8j+7 in memory order -> half(q * d): a sign-flipped byte (q + 128) under the
// exponent byte of 1024.0 is 1024 + 128 + q exactly; one subtract, one multiply (a single rounding).
__device__ __forceinline__ void dq_op_q8(int op, const Q8BlockRaw& blk, int j, half2v d2, DqTmp& tmp, U4& out) {
    const half2v k1152 = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    switch (op) {
        case 0: tmp.qa = blk.q[2 * j] ^ 0x80808080u; break;
        case 1: tmp.q8 = blk.q[2 * j + 1] ^ 0x80808080u; break;
        case 2: tmp.t[0] = as_h2(__builtin_amdgcn_perm(0x64646464u, tmp.qa, 0x04010400u)); break;
        case 3: tmp.t[1] = as_h2(__builtin_amdgcn_perm(0x64646464u, tmp.qa, 0x04030402u)); break;
        case 4: tmp.t[2] = as_h2(__builtin_amdgcn_perm(0x64646464u, tmp.q8, 0x04010400u)); break;
        case 5: tmp.t[3] = as_h2(__builtin_amdgcn_perm(0x64646464u, tmp.q8, 0x04030402u)); break;
        case 6: case 7: case 8: case 9: tmp.t[op - 6] -= k1152; break;
        default: out.v[op - 10] = as_u32(tmp.t[op - 10] * d2); break;
    }
}

// Q3 -> half(q * d + b), q = low2 | high << 2, in the same pair order as Q4: pair p of
// instruction j is weights 8j + p and 8j + p + 4.  One byte permute puts the two-bit fields of the
// first four weights in bits 0..7 and of the last four in bits 16..23, where a mantissa of
// 1024 / 4^p counts field p of each half in units of one; the high plane's byte of the same weights
// is spread to bits p and 16 + p once per instruction and shifted to bit 2p + 2 of each half per
// pair (units of four).
__device__ __forceinline__ void dq_op_q3(int op, const Q3BlockRaw& blk, int j, half2v d2, half2v b2, DqTmp& tmp,
                                         U4& out) {
    if (op == 0) {
        tmp.qa = __builtin_amdgcn_perm(0u, blk.lo[j >> 1], (j & 1) ? 0x0c030c02u : 0x0c010c00u);
    } else if (op == 1) {
        tmp.q8 = (blk.hi >> (8 * j)) & 0xffu;
    } else if (op == 2) {
        tmp.q8 = (tmp.q8 << 12) | tmp.q8;
    } else if (op == 3) {
        tmp.q8 &= 0x000F000Fu;  // bits p and 16 + p: high bits of weights 8j + p and 8j + p + 4
    } else {
        // stage by stage over the four pairs, so that no step waits on the one before it
        const int step = (op - 4) / 4, p = (op - 4) % 4;
        const uint32_t magic = p == 0 ? 0x64006400u : p == 1 ? 0x5C005C00u : p == 2 ? 0x54005400u : 0x4C004C00u;
        const _Float16 mv = static_cast<_Float16>(p == 0 ? 1024.0f : p == 1 ? 256.0f : p == 2 ? 64.0f : 16.0f);
        const half2v km = {mv, mv};
        switch (step) {
            case 0: tmp.t[p] = as_h2((tmp.qa & (0x00030003u << (2 * p))) | magic); break;
            case 1: out.v[p] = tmp.q8 << (p + 2); break;  // out.v[p] is free until the pair's last step
            case 2: tmp.t[p] = as_h2((out.v[p] & (0x00040004u << (2 * p))) | as_u32(tmp.t[p])); break;
            case 3: tmp.t[p] -= km; break;
            default: out.v[p] = as_u32(__builtin_elementwise_fma(tmp.t[p], d2, b2)); break;
        }
    }
}

template <int FMT, typename WBlock>
__device__ __forceinline__ void dq_op(int op, const WBlock& blk, int j, half2v d2, half2v b2, DqTmp& tmp, U4& out) {
    if constexpr (FMT == 0) dq_op_q4(op, blk.q[j], d2, b2, tmp, out);
    else if constexpr (FMT == 1) dq_op_q8(op, blk, j, d2, tmp, out);
    else dq_op_q3(op, blk, j, d2, b2, tmp, out);
}

// Eight consecutive f16 activations x0..x7 (as four dwords) -> x0 x4 x1 x5 x2 x6 x3 x7.
__device__ __forceinline__ uint4 interleave8(uint4 c) {
    uint4 r;
    r.x = __builtin_amdgcn_perm(c.z, c.x, 0x05040100u);
    r.y = __builtin_amdgcn_perm(c.z, c.x, 0x07060302u);
    r.z = __builtin_amdgcn_perm(c.w, c.y, 0x05040100u);
    r.w = __builtin_amdgcn_perm(c.w, c.y, 0x07060302u);
    return r;
}

__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {
    half2v h = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
    return as_u32(h);
}

// LORA: compiled with the LoRA step (kept out of the plain kernel, whose register allocation it
// would disturb).
//
// Scheduling.  Tiles are long (K/128 steps of ~2 us) and there is one per CU at a time, so a last,
// partly filled round of tiles would idle most of the chip for a whole tile time.  The launch
// therefore runs the first `full` tiles (a multiple of the CU count) whole, and cuts each of the
// remaining "tail" tiles into `tail_slices` K slices that run as separate, shorter workgroups
// (dispatched last).  A slice writes its 128 x 256 partial tile to scratch; gemm_reduce_tail adds
// the slices in slice order (deterministic) and applies the LoRA delta of those tiles in f32.
struct WregPlan {
    uint32_t full;         // tiles computed whole, written straight to y
    uint32_t tail_slices;  // K slices per remaining tile (1 = no slicing, written straight to y)
    float* partial;        // [tail tile][slice][TM * TN] when tail_slices > 1
};

// FMT: 0 = Q4 blocks, 1 = Q8_0, 2 = Q3 (the siblings have no LoRA step; Q8_0 keeps its activations in
// memory order, the other two in the x0 x4 x1 x5 .. order of their decoders).
template <bool X_F16, bool LORA, int FMT = 0>
__global__ __launch_bounds__(256, 1) void gemm_q4_wreg(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                       const void* __restrict__ xv, uint32_t m,
                                                       float* __restrict__ y, LoraEpilogue lora, WregPlan plan) {
    extern __shared__ uint4 lds16[];  // two activation buffers of kBuf16 units
    constexpr int XU = TM * (TK / 8) / 256;  // 8-activation units staged per thread per step
    constexpr int XL = X_F16 ? 1 : 2;        // 16-byte global loads per unit
    typedef typename WBlockOf<FMT>::type WBlock;
    constexpr uint32_t kBytes = WBlockOf<FMT>::kBytes;
    constexpr int kDqOps = DqOps<FMT>::kOps;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 15;  // row inside a 16-row tile
    const int g = lane >> 4;   // K group: block g of the step

    // ---- tile id -> (token tile, weight tile), grouped so co-resident tiles share activations
    // workgroup -> (tile, K slice): whole tiles first, then the slices of the tail tiles
    const bool in_tail = blockIdx.x >= plan.full;
    const uint32_t tail_idx = in_tail ? blockIdx.x - plan.full : 0;
    const uint32_t tile = in_tail ? plan.full + tail_idx / plan.tail_slices : blockIdx.x;
    const uint32_t nslices = in_tail ? plan.tail_slices : 1;
    const uint32_t slice = in_tail ? tail_idx % plan.tail_slices : 0;

    const uint32_t tiles_m = (m + TM - 1) / TM, tiles_n = (n + TN - 1) / TN;
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = tile / per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t group_m = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
    const uint32_t in_group = tile - group * per_group;
    const uint32_t m0 = (first_m + in_group % group_m) * TM;
    const uint32_t n0 = (in_group / group_m) * TN;

    // K slice of this workgroup (the whole row when nslices == 1).  From here on steps, blocks and
    // K offsets are counted from the start of the slice.
    const uint32_t nb_total = k / kBlockWeights;
    const uint32_t steps_total = (nb_total + 3) / 4;
    const uint32_t steps_per = (steps_total + nslices - 1) / nslices;
    const uint32_t s_begin = slice * steps_per;  // the host never plans an empty slice
    const uint32_t nsteps = s_begin + steps_per < steps_total ? steps_per : steps_total - s_begin;
    const uint32_t nb = nb_total - s_begin * 4;  // blocks from the slice start to the end of the row
    const uint32_t k_rem = k - s_begin * TK;
    const bool to_partial = nslices > 1;
    float* const ptile = to_partial ? plan.partial + (static_cast<size_t>(tile - plan.full) * nslices + slice) * (TM * TN)
                                    : nullptr;

    float4v acc[NU][NT];
#pragma unroll
    for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[u][t] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- per-thread global pointers -----------------------------------------------------------
    // first block of the slice in the lane's weight row of tile u; counted in dwords where the format's
    // blocks are whole dwords, in 2-byte units for Q8_0
    typedef typename std::conditional<FMT == 1, uint16_t, uint32_t>::type WUnit;
    constexpr uint32_t kUnits = kBytes / sizeof(WUnit);
    const WUnit* w_row[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        uint32_t row = n0 + wave * 64 + u * 16 + lr;
        row = row < n ? row : n - 1;
        w_row[u] = reinterpret_cast<const WUnit*>(w) + static_cast<size_t>(row) * (nb_total * kUnits) + s_begin * (4 * kUnits);
    }
    // activation unit i of this thread: token row tid/16 + 16 i, K offset 8 * (tid % 16) of the step
    const int x_part = tid & 15;
    const uint8_t* x_row[XU];
#pragma unroll
    for (int i = 0; i < XU; ++i) {
        uint32_t row = m0 + (tid >> 4) + 16 * i;
        row = row < m ? row : m - 1;
        x_row[i] = static_cast<const uint8_t*>(xv) +
                   (static_cast<size_t>(row) * k + static_cast<size_t>(s_begin) * TK) * (X_F16 ? 2 : 4);
    }

    struct XRegs {
        uint4 c[XU][XL];
    };

    auto load_x_unit = [&](XRegs& xr, int i, uint32_t s) {
        uint32_t koff = s * TK + x_part * 8;
        koff = koff < k_rem ? koff : k_rem - 8;  // past the end of K: any valid address, weights there are zero
        const size_t byte_off = static_cast<size_t>(koff) * (X_F16 ? 2 : 4);
#pragma unroll
        for (int l = 0; l < XL; ++l)
            xr.c[i][l] = *reinterpret_cast<const uint4*>(x_row[i] + byte_off + 16 * l);
    };
    auto store_x_unit = [&](const XRegs& xr, int i, uint4* buf) {
        uint4 out;
        if (X_F16) {
            out = FMT == 1 ? xr.c[i][0] : interleave8(xr.c[i][0]);
        } else if (FMT == 1) {
            const uint4 a = xr.c[i][0], b = xr.c[i][XL - 1];
            out.x = pack_h2(__builtin_bit_cast(float, a.x), __builtin_bit_cast(float, a.y));
            out.y = pack_h2(__builtin_bit_cast(float, a.z), __builtin_bit_cast(float, a.w));
            out.z = pack_h2(__builtin_bit_cast(float, b.x), __builtin_bit_cast(float, b.y));
            out.w = pack_h2(__builtin_bit_cast(float, b.z), __builtin_bit_cast(float, b.w));
        } else {
            const uint4 a = xr.c[i][0], b = xr.c[i][XL - 1];
            out.x = pack_h2(__builtin_bit_cast(float, a.x), __builtin_bit_cast(float, b.x));
            out.y = pack_h2(__builtin_bit_cast(float, a.y), __builtin_bit_cast(float, b.y));
            out.z = pack_h2(__builtin_bit_cast(float, a.z), __builtin_bit_cast(float, b.z));
            out.w = pack_h2(__builtin_bit_cast(float, a.w), __builtin_bit_cast(float, b.w));
        }
        buf[((tid >> 4) + 16 * i) * kPitch16 + x_part] = out;
    };
    auto load_w_one = [&](WBlock (&wr)[NU], uint32_t s, int u) {
        uint32_t blk = s * 4 + g;
        blk = blk < nb ? blk : nb - 1;
        wr[u] = *reinterpret_cast<const WBlock*>(w_row[u] + blk * kUnits);
    };
    auto load_w = [&](WBlock (&wr)[NU], uint32_t s) {
#pragma unroll
        for (int u = 0; u < NU; ++u) load_w_one(wr, s, u);
    };

    auto scale_pair = [&](const WBlock& blk, bool live, half2v& d2, half2v& b2) {
        uint32_t sb;
        if constexpr (FMT == 1) sb = live ? static_cast<uint32_t>(blk.d) : 0u;  // scale only
        else sb = live ? blk.sb : 0u;
        d2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x01000100u));  // (d, d)
        b2 = as_h2(__builtin_amdgcn_perm(sb, sb, 0x03020302u));  // (b, b)
    };

    // State carried from step to step: the dequantised weights of the coming step's first
    // quarter and the (scale, bias) pairs of the coming step's blocks.
    U4 a_cur[NU];
    half2v d2[NU], b2[NU];
    XRegs xr;

    // One K step = 4 quarters x 8 token tiles x 4 weight tiles = 128 matrix-core instructions,
    // issued in a fixed order.  In the shadow of each instruction go one or two steps of the
    // dequantisation of the NEXT quarter (for the last quarter: the first quarter of step s+1,
    // from `wnext`), and every fourth token tile one activation unit of step s+1 is written to the
    // other LDS buffer and refilled from global memory for step s+2.  LDS operand reads run two
    // token tiles ahead.  `wfree` was consumed in the previous step and is refilled for step s+2
    // during the first quarter.
    auto step = [&](uint32_t s, WBlock (&wr)[NU], WBlock (&wnext)[NU], WBlock (&wfree)[NU]) {
        const uint4* xbuf = lds16 + (s & 1) * kBuf16 + lr * kPitch16 + 4 * g;
        uint4* xnext = lds16 + ((s + 1) & 1) * kBuf16;
        const bool live_next = (s + 1) * 4 + g < nb;
        half2v d2n[NU], b2n[NU];
        U4 a_nxt[NU];
        DqTmp tmp;
        uint4 bx[3];
        bx[0] = xbuf[0];
        bx[1] = xbuf[16 * kPitch16];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const int p = j * NT + t;  // slot: (quarter, token tile)
                // one weight tile's loads every other token tile rather than all eight at the step's
                // start: a burst from every wave right after the barrier fills the address unit's queue
                if (j == 0 && (t & 1) == 0) load_w_one(wfree, s + 2, t / 2);
                if (p + 2 < 4 * NT) {
                    const int pj = (p + 2) / NT, pt = (p + 2) % NT;
                    bx[(p + 2) % 3] = xbuf[pt * 16 * kPitch16 + pj];
                }
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const int c = t * NU + u;  // instruction index inside the quarter, 0..31
                    acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, a_cur[u]), __builtin_bit_cast(half8, bx[p % 3]), acc[u][t], 0, 0,
                        0);
#pragma unroll
                    for (int e = c * (NU * kDqOps) / 32; e < (c + 1) * (NU * kDqOps) / 32; ++e) {
                        const int uu = e / kDqOps, op = e % kDqOps;
                        if (j < 3) dq_op<FMT>(op, wr[uu], j + 1, d2[uu], b2[uu], tmp, a_nxt[uu]);
                        else dq_op<FMT>(op, wnext[uu], 0, d2n[uu], b2n[uu], tmp, a_nxt[uu]);
                    }
                    if (j == 2 && t == NT - 1) scale_pair(wnext[u], live_next, d2n[u], b2n[u]);
                    if (u == NU - 1 && (p & 3) == 1) {
                        store_x_unit(xr, p >> 2, xnext);
                        load_x_unit(xr, p >> 2, s + 2);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int u = 0; u < NU; ++u) a_cur[u] = a_nxt[u];
        }
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            d2[u] = d2n[u];
            b2[u] = b2n[u];
        }
        __syncthreads();
    };

    WBlock wa[NU], wb[NU], wc[NU];
#pragma unroll
    for (int i = 0; i < XU; ++i) load_x_unit(xr, i, 0);
    load_w(wa, 0);
    load_w(wb, 1);
#pragma unroll
    for (int i = 0; i < XU; ++i) {
        store_x_unit(xr, i, lds16);
        load_x_unit(xr, i, 1);
    }
    {
        DqTmp tmp;
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            scale_pair(wa[u], g < nb, d2[u], b2[u]);
#pragma unroll
            for (int op = 0; op < kDqOps; ++op) dq_op<FMT>(op, wa[u], 0, d2[u], b2[u], tmp, a_cur[u]);
        }
    }
    __syncthreads();

    uint32_t s = 0;
    for (; s + 3 <= nsteps; s += 3) {
        step(s, wa, wb, wc);
        step(s + 1, wb, wc, wa);
        step(s + 2, wc, wa, wb);
    }
    if (s < nsteps) step(s, wa, wb, wc);
    if (s + 1 < nsteps) step(s + 1, wb, wc, wa);

    // ---- LoRA: one more K step of depth `rank` on the matrix cores,
    //      acc[n, token] += sum_r B[n, r] * (scale * t[token, r]).
    // Both factors are split hi + lo/2048 into f16 so the delta keeps f32-level accuracy:
    // B.t = Bhi.thi + (Bhi/2048).tlo + Blo.(thi/2048); the last term vanishes for f16-stored B.
    if (LORA && lora.rank && !to_partial) {
        for (uint32_t r0 = 0; r0 < lora.rank; r0 += 32) {
            const uint32_t rbase = r0 + 8 * g;  // this lane's eight rank indices
            half8 b_hi[NU], b_his[NU], b_lo[NU];
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                uint32_t row = n0 + wave * 64 + u * 16 + lr;
                row = row < n ? row : n - 1;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t idx = rbase + i;
                    const float bv =
                        idx < lora.rank ? load_b(lora.b, lora.b_is_f16, static_cast<size_t>(row) * lora.rank + idx) : 0.0f;
                    const _Float16 hi = static_cast<_Float16>(bv);
                    b_hi[u][i] = hi;
                    b_his[u][i] = static_cast<_Float16>(bv * (1.0f / 2048.0f));
                    b_lo[u][i] = static_cast<_Float16>((bv - static_cast<float>(hi)) * 2048.0f);
                }
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                uint32_t tok = m0 + t * 16 + lr;
                tok = tok < m ? tok : m - 1;
                half8 t_hi, t_his, t_lo;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t idx = rbase + i;
                    const float tv = idx < lora.rank ? lora.scale * lora.t[static_cast<size_t>(tok) * lora.rank + idx] : 0.0f;
                    const _Float16 hi = static_cast<_Float16>(tv);
                    t_hi[i] = hi;
                    t_his[i] = static_cast<_Float16>(tv * (1.0f / 2048.0f));
                    t_lo[i] = static_cast<_Float16>((tv - static_cast<float>(hi)) * 2048.0f);
                }
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b_hi[u], t_hi, acc[u][t], 0, 0, 0);
                    acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b_his[u], t_lo, acc[u][t], 0, 0, 0);
                    if (!lora.b_is_f16)
                        acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b_lo[u], t_his, acc[u][t], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: element v of lane l of a 16x16 result is weight row 4*(l/16) + v, token l%16
    const bool vec_ok = (n & 3u) == 0;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const uint32_t gn = n0 + wave * 64 + u * 16 + 4 * g;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const uint32_t gm = m0 + t * 16 + lr;
            if (gm >= m || gn >= n) continue;
            const float4v val = acc[u][t];
            if (to_partial) {  // tile-local layout, always 16-byte aligned
                *reinterpret_cast<float4v*>(ptile + (gm - m0) * TN + (gn - n0)) = val;
                continue;
            }
            float* dst = y + static_cast<size_t>(gm) * n + gn;
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

// ---- two workgroups per CU: activations packed ahead of time, loaded straight into LDS ------------
//
// The kernel above holds 400 registers per lane (one wave per SIMD), and a wave alone cannot issue
// matrix-core instructions back to back: its own dequantisation, LDS reads and waits sit between
// them.  gemm_q4_w2 is the same tile and the same instruction order within 256 registers, so that
// two workgroups share a CU and one wave's gaps are the other's issue slots.  What makes room:
//  * the activations arrive already converted to f16, in the dequantiser's pair order and in the
//    tile order of LDS (pack_x_tiles_kernel, one pass over X per call), so a K step's 32 KB go from
//    global memory to LDS with eight global_load_lds_dwordx4 per wave: no staging registers, no
//    permutes and no LDS stores in the loop;
//  * two rotating weight register sets instead of three: the set of step s is dead once its last
//    quarter has been dequantised (in the shadow of quarter 2) and is refilled for step s + 2 at the
//    start of quarter 3.
// LDS holds a step's activations as [token tile 8][K chunk 16][token 16] units of 16 bytes (8 f16), the
// order packed X has in memory: the 16 lanes of a lane group read 256 contiguous bytes.
constexpr int kStepUnits = TM * (TK / 8);  // 16-byte units of activations per K step: 2048 = 32 KB

// dq_op_q4 with scale and bias taken straight from the block's first dword (d in the low half, b in
// the high half) through the packed fma's operand selectors: no (d, d) / (b, b) registers.
__device__ __forceinline__ uint32_t pk_fma_sb(half2v t, uint32_t sb) {
    uint32_t r;
    asm("v_pk_fma_f16 %0, %1, %2, %2 op_sel:[0,0,1] op_sel_hi:[1,0,1]" : "=v"(r) : "v"(t), "v"(sb));
    return r;
}
__device__ __forceinline__ void dq_op_q4_sb(int op, uint32_t q, uint32_t sb, DqTmp& tmp, U4& out) {
    if (op < 9) dq_op_q4(op, q, half2v{}, half2v{}, tmp, out);
    else out.v[op - 9] = pk_fma_sb(tmp.t[op - 9], sb);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int OFF>
__device__ __forceinline__ u32x4 lds_read128(uint32_t addr) {
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF) : "memory");
    return r;
}
// Waits until at most N LDS operations of the wave are outstanding; `r` is the register the wait is
// for, so that no use of it can move ahead of the wait.
template <int N>
__device__ __forceinline__ void lds_wait(u32x4& r) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(r) : "n"(N));
}
// acc += A . B on the matrix cores with the accumulator pinned to the accumulation registers: the
// 128 accumulators of a wave then never compete with the loop's working set for the 128 ordinary
// vector registers that two waves per SIMD leave each wave.  Every accumulator is touched once per
// quarter (32 instructions apart), so no two dependent instructions are back to back.
__device__ __forceinline__ void mfma_in_place(float4v& c, const U4& a, const u32x4& b) {
    const u32x4 av = {a.v[0], a.v[1], a.v[2], a.v[3]};
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(av), "v"(b));
}

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void global_void_t;

// X [m, k] (f16 or f32, row-major) -> f16 units [token tile][K chunk of 8][token in tile 16][8], the 8
// in the order x0 x4 x1 x5 x2 x6 x3 x7; token tiles up to a multiple of 8 and K chunks up to
// kc_pad (a multiple of 16) are zero-filled.  One thread per unit.
__global__ __launch_bounds__(256) void pack_x_tiles_kernel(const void* __restrict__ xv, int x_is_f16, uint32_t m,
                                                           uint32_t k, uint32_t kc_pad, uint4* __restrict__ out,
                                                           uint64_t units) {
    const uint64_t u = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (u >= units) return;
    const uint32_t lr = static_cast<uint32_t>(u & 15);
    const uint64_t rest = u >> 4;
    const uint32_t kc = static_cast<uint32_t>(rest % kc_pad);
    const uint32_t row = static_cast<uint32_t>(rest / kc_pad) * 16 + lr;
    uint4 r = {0u, 0u, 0u, 0u};
    if (row < m && kc * 8 < k) {
        if (x_is_f16) {
            r = interleave8(*reinterpret_cast<const uint4*>(static_cast<const _Float16*>(xv) + static_cast<size_t>(row) * k + kc * 8));
        } else {
            const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(xv) + static_cast<size_t>(row) * k + kc * 8);
            const float4 a = p[0], b = p[1];
            r.x = pack_h2(a.x, b.x);
            r.y = pack_h2(a.y, b.y);
            r.z = pack_h2(a.z, b.z);
            r.w = pack_h2(a.w, b.w);
        }
    }
    out[u] = r;
}

__global__ __launch_bounds__(256, 2) void gemm_q4_w2(const uint8_t* __restrict__ w, uint32_t n, uint32_t k,
                                                     const uint4* __restrict__ xp, uint32_t kc_pad, uint32_t m,
                                                     float* __restrict__ y, WregPlan plan) {
    extern __shared__ uint4 lds16[];  // two activation buffers of kStepUnits units
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lr = lane & 15;  // row inside a 16-row tile
    const int g = lane >> 4;   // K group: block g of the step

    // ---- workgroup -> (tile, K slice).  Whole tiles first, then the slices of the tail tiles; inside
    // either range, workgroups that land on one XCD (blockIdx % 8) take a contiguous run of tile ids,
    // i.e. neighbouring weight tiles: each XCD's L2 then streams an eighth of W instead of all of it.
    const uint32_t n_whole = plan.full, n_tail = gridDim.x - plan.full;
    const bool in_tail = blockIdx.x >= n_whole;
    const uint32_t pos = in_tail ? blockIdx.x - n_whole : blockIdx.x, count = in_tail ? n_tail : n_whole;
    const uint32_t xcd = pos & 7u, per = count >> 3, rem = count & 7u;
    const uint32_t item = xcd * per + (xcd < rem ? xcd : rem) + (pos >> 3);
    const uint32_t tile = in_tail ? plan.full + item / plan.tail_slices : item;
    const uint32_t nslices = in_tail ? plan.tail_slices : 1;
    const uint32_t slice = in_tail ? item % plan.tail_slices : 0;

    const uint32_t tiles_m = (m + TM - 1) / TM, tiles_n = (n + TN - 1) / TN;
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = tile / per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t group_m = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
    const uint32_t in_group = tile - group * per_group;
    const uint32_t m0 = (first_m + in_group % group_m) * TM;
    const uint32_t n0 = (in_group / group_m) * TN;

    const uint32_t nb_total = k / kBlockWeights;
    const uint32_t steps_total = (nb_total + 3) / 4;
    const uint32_t steps_per = (steps_total + nslices - 1) / nslices;
    const uint32_t s_begin = slice * steps_per;  // the host never plans an empty slice
    const uint32_t nsteps = s_begin + steps_per < steps_total ? steps_per : steps_total - s_begin;
    const uint32_t nb = nb_total - s_begin * 4;  // blocks from the slice start to the end of the row
    const bool to_partial = nslices > 1;
    float* const ptile = to_partial ? plan.partial + (static_cast<size_t>(tile - plan.full) * nslices + slice) * (TM * TN)
                                    : nullptr;

    float4v acc[NU][NT];
#pragma unroll
    for (int u = 0; u < NU; ++u)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[u][t] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

    // byte offset of the lane's weight row of tile u from the first block of the slice in row 0 (rows
    // past the end are clamped to the last row: their results are never stored); a uniform base plus
    // 32-bit lane offsets keeps the addresses in 4 registers (a Q4 tensor is far below 4 GB)
    const uint8_t* const w_base = w + static_cast<size_t>(s_begin) * (4 * kBlockBytes);
    uint32_t w_off[NU];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        uint32_t row = n0 + wave * 64 + u * 16 + lr;
        row = row < n ? row : n - 1;
        w_off[u] = row * (nb_total * static_cast<uint32_t>(kBlockBytes));
    }
    auto load_w_one = [&](Q4BlockRaw (&wr)[NU], uint32_t s, int u) {
        uint32_t blk = s * 4 + g;
        blk = blk < nb ? blk : nb - 1;
        wr[u] = *reinterpret_cast<const Q4BlockRaw*>(w_base + (w_off[u] + blk * static_cast<uint32_t>(kBlockBytes)));
    };
    auto load_w = [&](Q4BlockRaw (&wr)[NU], uint32_t s) {
#pragma unroll
        for (int u = 0; u < NU; ++u) load_w_one(wr, s, u);
    };

    // The activations of step s of this slice: token tile i of the workgroup is 4 KB contiguous in packed X
    // and in LDS; wave w moves its quarter (64 units) of each of the 8 token tiles.  Steps past the
    // slice re-read its last step, so that every step issues the same eight loads.
    const uint4* const x_src = xp + (static_cast<size_t>(m0 / 16) * kc_pad + static_cast<size_t>(s_begin) * 16) * 16 + wave * 64 + lane;
    auto load_x_one = [&](uint32_t s, int buf, int i) {
        const uint32_t ss = s < nsteps ? s : nsteps - 1;
        const uint4* src = x_src + static_cast<size_t>(ss) * 256;
        uint4* dst = lds16 + buf * kStepUnits + wave * 64;
        __builtin_amdgcn_global_load_lds((global_void_t*)(src + static_cast<size_t>(i) * kc_pad * 16),
                                         (lds_void_t*)(dst + i * 256), 16, 0, 0);
    };
    auto load_x = [&](uint32_t s, int buf) {
#pragma unroll
        for (int i = 0; i < NT; ++i) load_x_one(s, buf, i);
    };

    U4 a_cur[NU];

    // One K step, the instruction order of gemm_q4_wreg: 4 quarters x 8 token tiles x 4 weight tiles,
    // in the shadow of each matrix-core instruction one or two steps of the next quarter's
    // dequantisation, LDS operand reads two token tiles ahead.  `wr` holds this step's blocks and is
    // refilled for step s + 2 when its last quarter has been dequantised; `wnext` holds step s + 1.
    // The operand reads are written as ds_read_b128 by hand, with their waits: a read the compiler
    // knows of is made to wait for every global_load_lds in flight (it cannot tell the two LDS
    // buffers apart), which would stall each step on the activations of the next.
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char*)lds16));
    auto step = [&](uint32_t s, Q4BlockRaw (&wr)[NU], Q4BlockRaw (&wnext)[NU]) {
        const uint32_t xaddr = lds_base + ((s & 1) * kStepUnits + (4 * g) * 16 + lr) * 16;
        const bool live_next = (s + 1) * 4 + g < nb;
        U4 a_nxt[NU];
        DqTmp tmp;
        u32x4 bx[3];
        bx[0] = lds_read128<0>(xaddr);
        bx[1] = lds_read128<256 * 16>(xaddr);
        __builtin_amdgcn_sched_barrier(0);
        static_for<4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            static_for<NT>([&](auto tc) {
                constexpr int t = decltype(tc)::value;
                constexpr int p = j * NT + t;  // slot: (quarter, token tile)
                // Memory instructions one at a time between the token tiles: a burst of them from all
                // eight waves right after the barrier would fill the address unit's queue, and a wave
                // whose load is not accepted cannot issue its matrix instructions either.
                if constexpr (j == 0) load_x_one(s + 1, (s + 1) & 1, t);  // next step's activations, token tile t
                if constexpr (j == 3 && (t & 1) == 0) load_w_one(wr, s + 2, t / 2);  // wr is free: refill for step s + 2
                if constexpr (p + 2 < 4 * NT) {
                    constexpr int pj = (p + 2) / NT, pt = (p + 2) % NT;
                    bx[(p + 2) % 3] = lds_read128<(pt * 256 + pj * 16) * 16>(xaddr);
                }
                // the read of slot p is done when at most the reads of slots p + 1 and p + 2 are out
                lds_wait<(p + 2 < 4 * NT) ? 2 : (4 * NT - 1 - p)>(bx[p % 3]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const int c = t * NU + u;  // instruction index inside the quarter, 0..31
                    mfma_in_place(acc[u][t], a_cur[u], bx[p % 3]);
#pragma unroll
                    for (int e = c * (NU * 13) / 32; e < (c + 1) * (NU * 13) / 32; ++e) {
                        const int uu = e / 13, op = e % 13;
                        if (j < 3) dq_op_q4_sb(op, wr[uu].q[j + 1], wr[uu].sb, tmp, a_nxt[uu]);
                        else dq_op_q4_sb(op, wnext[uu].q[0], wnext[uu].sb, tmp, a_nxt[uu]);
                    }
                    if (j == 2 && t == NT - 1) wnext[u].sb = live_next ? wnext[u].sb : 0u;  // a block past the end of K counts as zero
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
#pragma unroll
            for (int u = 0; u < NU; ++u) a_cur[u] = a_nxt[u];
        });
        // the activations of step s + 1 have landed (only the weight loads of step s + 2, issued after
        // them, may still be in flight), and every wave is done reading this step's buffer
        asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
    };

    Q4BlockRaw wa[NU], wb[NU];
    load_x(0, 0);
    load_w(wa, 0);
    load_w(wb, 1);
    {
        DqTmp tmp;
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            wa[u].sb = static_cast<uint32_t>(g) < nb ? wa[u].sb : 0u;
#pragma unroll
            for (int op = 0; op < 13; ++op) dq_op_q4_sb(op, wa[u].q[0], wa[u].sb, tmp, a_cur[u]);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");

    uint32_t s = 0;
    for (; s + 2 <= nsteps; s += 2) {
        step(s, wa, wb);
        step(s + 1, wb, wa);
    }
    if (s < nsteps) step(s, wa, wb);
    // the last matrix-core results are 8 passes from their registers
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: element v of lane l of a 16x16 result is weight row 4*(l/16) + v, token l%16
    const bool vec_ok = (n & 3u) == 0;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const uint32_t gn = n0 + wave * 64 + u * 16 + 4 * g;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const uint32_t gm = m0 + t * 16 + lr;
            if (gm >= m || gn >= n) continue;
            const float4v val = acc[u][t];
            if (to_partial) {  // tile-local layout, always 16-byte aligned
                *reinterpret_cast<float4v*>(ptile + (gm - m0) * TN + (gn - n0)) = val;
                continue;
            }
            float* dst = y + static_cast<size_t>(gm) * n + gn;
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

// Sums the K slices of the tail tiles in slice order and writes them to y, adding the LoRA delta
// scale * sum_j B[row, j] * t[token, j] in f32.  grid (tail tiles, TM * TN / 1024); a thread owns four
// consecutive weight rows of one token.
__global__ __launch_bounds__(256) void gemm_reduce_tail(const float* __restrict__ partial, uint32_t first_tile,
                                                        uint32_t slices, uint32_t m, uint32_t n,
                                                        float* __restrict__ y, LoraEpilogue lora) {
    const uint32_t tile = first_tile + blockIdx.x;
    const uint32_t tiles_m = (m + TM - 1) / TM, tiles_n = (n + TN - 1) / TN;
    const uint32_t per_group = kGroupM * tiles_n;
    const uint32_t group = tile / per_group;
    const uint32_t first_m = group * kGroupM;
    const uint32_t group_m = tiles_m - first_m < kGroupM ? tiles_m - first_m : kGroupM;
    const uint32_t in_group = tile - group * per_group;
    const uint32_t m0 = (first_m + in_group % group_m) * TM;
    const uint32_t n0 = (in_group / group_m) * TN;

    const uint32_t local = (blockIdx.y * 256 + threadIdx.x) * 4;  // element index inside the tile
    const uint32_t lrow = local / TN, lcol = local % TN;
    const uint32_t token = m0 + lrow, row = n0 + lcol;
    if (token >= m || row >= n) return;
    const float* src = partial + static_cast<size_t>(blockIdx.x) * slices * (TM * TN) + local;
    float4v v = *reinterpret_cast<const float4v*>(src);
    for (uint32_t sl = 1; sl < slices; ++sl) v += *reinterpret_cast<const float4v*>(src + static_cast<size_t>(sl) * (TM * TN));
    if (lora.rank) {
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        const float* t = lora.t + static_cast<size_t>(token) * lora.rank;
        float4v d = {0.0f, 0.0f, 0.0f, 0.0f};
        if ((lora.rank & 3u) == 0) {  // t[token, :] is a broadcast load, the B rows are read with vector loads
            for (uint32_t j = 0; j < lora.rank; j += 4) {
                const float4v tv = *reinterpret_cast<const float4v*>(t + j);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t r = row + e < n ? row + e : n - 1;
                    const size_t bi = static_cast<size_t>(r) * lora.rank + j;
                    float4v bv;
                    if (lora.b_is_f16) {
                        const half4v h = *reinterpret_cast<const half4v*>(static_cast<const _Float16*>(lora.b) + bi);
                        bv = float4v{static_cast<float>(h[0]), static_cast<float>(h[1]), static_cast<float>(h[2]),
                                     static_cast<float>(h[3])};
                    } else {
                        bv = *reinterpret_cast<const float4v*>(static_cast<const float*>(lora.b) + bi);
                    }
                    d[e] = fmaf(bv[3], tv[3], fmaf(bv[2], tv[2], fmaf(bv[1], tv[1], fmaf(bv[0], tv[0], d[e]))));
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t r = row + e < n ? row + e : n - 1;
                for (uint32_t j = 0; j < lora.rank; ++j)
                    d[e] = fmaf(load_b(lora.b, lora.b_is_f16, static_cast<size_t>(r) * lora.rank + j), t[j], d[e]);
            }
        }
        v += lora.scale * d;
    }
    float* dst = y + static_cast<size_t>(token) * n + row;
    if ((n & 3u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0) {
        *reinterpret_cast<float4v*>(dst) = v;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (row + e < n) dst[e] = v[e];
    }
}

constexpr uint32_t kCus = 256;
constexpr uint32_t kMaxTailSlices = 16;
// Cost of one K slice of one tail tile, in K steps of a tile: its 128 KB partial tile is written and
// read back once (~0.06 us of memory time against ~2.4 us per step).
#ifndef LQ4_SLICE_CHARGE
#define LQ4_SLICE_CHARGE 0.027
#endif

// How the tiles of a shape are scheduled: `full` whole tiles, the rest in `slices` K slices each.
struct HostPlan {
    uint32_t tiles, full, slices;
};

HostPlan plan_tiles(uint32_t n, uint32_t k, uint32_t m, uint32_t slots = kCus) {
    const uint32_t tiles = ((n + TN - 1) / TN) * ((m + TM - 1) / TM);
    const uint32_t steps = (k / kBlockWeights + 3) / 4;
    const uint32_t rest = tiles % slots;
    HostPlan p{tiles, tiles - rest, 1};
    if (rest == 0 || steps < 4) return HostPlan{tiles, tiles, 1};
    // pick the slice count that minimises the time of the last round in K steps,
    // ceil(rest * s / CUs) * steps-per-slice plus the traffic of the partial tiles,
    // with at least two steps per slice and no empty slice
    double best = steps;  // s = 1: one round of whole tiles
    for (uint32_t s = 2; s <= kMaxTailSlices && s * 2 <= steps; ++s) {
        const uint32_t per = (steps + s - 1) / s;
        if ((s - 1) * per >= steps) continue;  // would leave the last slice empty
        const double rounds = static_cast<double>((rest * s + slots - 1) / slots);
        const double t = rounds * per + LQ4_SLICE_CHARGE * rest * s;
        if (t < best - 1e-9) {
            best = t;
            p.slices = s;
        }
    }
    if (p.slices == 1) p.full = tiles;
    return p;
}

}  // namespace

uint32_t gemm_wreg_tiles(uint32_t n, uint32_t m) { return ((n + TN - 1) / TN) * ((m + TM - 1) / TM); }

bool gemm_wreg_supports(uint32_t, uint32_t k, uint32_t, int) { return k >= kBlockWeights; }

// The two-workgroups-per-CU kernel pays one pass over X for packing and schedules in rounds of 512
// tiles: it is ahead (4-13 % measured) where there is at least one such round of whole tiles.
bool gemm_w2_wants(uint32_t n, uint32_t k, uint32_t m) {
    return k >= kBlockWeights && gemm_wreg_tiles(n, m) >= 2 * kCus;
}

size_t gemm_wreg_scratch_floats(uint32_t n, uint32_t k, uint32_t m) {
    const HostPlan p = plan_tiles(n, k, m);
    return p.slices > 1 ? static_cast<size_t>(p.tiles - p.full) * p.slices * (TM * TN) : 0;
}

namespace {

template <bool X_F16, bool LORA, int FMT>
void launch_wreg_t(const uint8_t* w, uint32_t n, uint32_t k, const void* x, uint32_t m, float* y,
                   const LoraEpilogue& lora, const HostPlan& hp, float* partial, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemm_q4_wreg<X_F16, LORA, FMT>), 160 * 1024);
    const size_t lds = 2 * kBuf16 * sizeof(uint4);
    const WregPlan plan{hp.full, hp.slices, partial};
    const uint32_t wgs = hp.full + (hp.tiles - hp.full) * hp.slices;
    hipLaunchKernelGGL((gemm_q4_wreg<X_F16, LORA, FMT>), dim3(wgs), dim3(256), lds, stream, w, n, k, x, m, y, lora,
                       plan);
}

}  // namespace

void launch_gemm_wreg(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m,
                      float* y, const LoraEpilogue& lora, float* partial, hipStream_t stream, int fmt) {
    HostPlan hp = plan_tiles(n, k, m);
    if (!partial) hp = HostPlan{hp.tiles, hp.tiles, 1};
    if (fmt == 1) {
        if (x_is_f16) launch_wreg_t<true, false, 1>(w, n, k, x, m, y, lora, hp, partial, stream);
        else launch_wreg_t<false, false, 1>(w, n, k, x, m, y, lora, hp, partial, stream);
    } else if (fmt == 2) {
        if (x_is_f16) launch_wreg_t<true, false, 2>(w, n, k, x, m, y, lora, hp, partial, stream);
        else launch_wreg_t<false, false, 2>(w, n, k, x, m, y, lora, hp, partial, stream);
    } else {
        // the matrix-core LoRA step serves the whole tiles; the tail tiles get their delta from the reduction
        const bool lora_in_kernel = lora.rank && hp.full > 0;
        if (lora_in_kernel) {
            if (x_is_f16) launch_wreg_t<true, true, 0>(w, n, k, x, m, y, lora, hp, partial, stream);
            else launch_wreg_t<false, true, 0>(w, n, k, x, m, y, lora, hp, partial, stream);
        } else {
            if (x_is_f16) launch_wreg_t<true, false, 0>(w, n, k, x, m, y, lora, hp, partial, stream);
            else launch_wreg_t<false, false, 0>(w, n, k, x, m, y, lora, hp, partial, stream);
        }
    }
    if (hp.slices > 1)
        hipLaunchKernelGGL(gemm_reduce_tail, dim3(hp.tiles - hp.full, TM * TN / 1024), dim3(256), 0, stream, partial,
                           hp.full, hp.slices, m, n, y, lora);
}

// ---- gemm_q4_w2: scratch = [packed X | partial tiles of the sliced tail] ----------------------------
namespace {
constexpr uint32_t kW2Slots = 2 * kCus;  // two workgroups per CU
inline uint32_t w2_kc_pad(uint32_t k) { return (k / 8 + 15) / 16 * 16; }
inline size_t w2_packed_bytes(uint32_t k, uint32_t m) {
    return static_cast<size_t>((m + TM - 1) / TM) * TM * w2_kc_pad(k) * 16;
}
}  // namespace

size_t gemm_w2_scratch_bytes(uint32_t n, uint32_t k, uint32_t m) {
    const HostPlan p = plan_tiles(n, k, m, kW2Slots);
    const size_t partial = p.slices > 1 ? static_cast<size_t>(p.tiles - p.full) * p.slices * (TM * TN) * sizeof(float) : 0;
    return w2_packed_bytes(k, m) + partial;
}

void launch_gemm_w2(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    uint8_t* scratch, hipStream_t stream) {
    const LoraEpilogue lora{nullptr, nullptr, 0, 0, 0.0f};  // no LoRA step in this kernel
    const HostPlan hp = plan_tiles(n, k, m, kW2Slots);
    const uint32_t kc_pad = w2_kc_pad(k);
    uint4* packed = reinterpret_cast<uint4*>(scratch);
    float* partial = reinterpret_cast<float*>(scratch + w2_packed_bytes(k, m));
    const uint64_t units = w2_packed_bytes(k, m) / 16;
    hipLaunchKernelGGL(pack_x_tiles_kernel, dim3(static_cast<uint32_t>((units + 255) / 256)), dim3(256), 0, stream, x,
                       x_is_f16, m, k, kc_pad, packed, units);
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemm_q4_w2), 64 * 1024);
    const size_t lds = 2 * kStepUnits * sizeof(uint4);
    const WregPlan plan{hp.full, hp.slices, partial};
    const uint32_t wgs = hp.full + (hp.tiles - hp.full) * hp.slices;
    hipLaunchKernelGGL(gemm_q4_w2, dim3(wgs), dim3(256), lds, stream, w, n, k, packed, kc_pad, m, y, plan);
    if (hp.slices > 1)
        hipLaunchKernelGGL(gemm_reduce_tail, dim3(hp.tiles - hp.full, TM * TN / 1024), dim3(256), 0, stream, partial,
                           hp.full, hp.slices, m, n, y, lora);
}

}  // namespace lq4
