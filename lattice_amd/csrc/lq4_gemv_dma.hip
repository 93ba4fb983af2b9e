// Batch-1 decode GEMV whose weights never pass through a register on their way in:  y[n] = sum_k W[n,k] * x[k].
//
// The lane-owns-block kernel (lq4_gemv_b1.hip) loads 20-byte blocks with a 16-byte and a 4-byte load per lane.
// That costs it twice: a wave's 16-byte loads at a 20-byte stride touch 1280 bytes for 1024 used (a read of the
// lm_head tensor in that pattern runs at 6.0 TB/s where dense 16-byte loads run at 6.7), and every load needs
// its 64-bit address formed in vector registers, which is vector issue the dot products then lack.
//
// Here a "slot" is one 64-block slab of one weight row, 1280 contiguous bytes, brought from memory straight into
// LDS by two dense loads (global_load_lds: lane l moves bytes 16 l .. 16 l + 15, then the 256 bytes behind them,
// 4 l .. 4 l + 3), so LDS holds the slab verbatim and lane l finds its block at byte 20 l.  Addresses are scalar
// arithmetic plus one fixed lane offset.  Each wave owns a ring of slots in LDS and keeps it full: requests run
// `ring` slots ahead of the arithmetic, across rows and chunks, and occupy no vector register.
//
// The compiler's wait-count pass knows nothing of these loads, so the waits are written by hand: a wave's loads
// return in the order they were issued, `s_waitcnt vmcnt(N)` with N = the number of load instructions issued
// after the slot at the head of the ring (two per slot) is exactly "the head has landed".  The y stores raise the
// same counter and may complete early, which can only make a wait longer than needed.  The activations are loaded
// by inline assembly too (ahead of the first weight request, so they are waited for alone) and staged in LDS as
// in the lane-owns-block kernel (lq4_b1_dev.hpp: per-block scaled fixed point, eight-wide 4-bit dot products).
//
// Every wave takes one run of consecutive rows, so its slots are one run of memory and the address of the next
// request is a running pointer.  The ring has a compile-time depth D and the loop is unrolled D times: the slot a
// wave has just emptied is the one its next request fills, so every LDS offset is a constant, the wait in the
// steady state is the constant vmcnt(2 (D - 1)), and what is left per slot is a dozen scalar instructions.  (A
// first version with run-time ring positions and a wait chosen by a switch spent ~80 scalar instructions and a
// dozen branches per slot and was 10-15 % slower than the lane-owns-block kernel: a CU issues one scalar
// instruction per cycle for all its waves.)  Shapes whose rows are 1, 2 or 3 whole slabs keep the lane's blocks of
// x in registers for the whole launch; other shapes (a short last slab, longer rows) re-read them from LDS.
#include "lq4_b1_dev.hpp"

namespace lq4 {

namespace {

using namespace b1;

constexpr int kSlotBytes = 1280;  // 64 blocks of 20 bytes

__device__ __forceinline__ uint32_t uniform(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

// By value on purpose: __builtin_bit_cast applied directly to an element of a vector (v.y) reads element 0.
__device__ __forceinline__ float as_f32(uint32_t bits) { return __builtin_bit_cast(float, bits); }

// Memory -> LDS, 16 or 4 bytes a lane: lane l's bytes land at LDS byte address `lds` + 16 l (or + 4 l).
// `base` and `lds` are wave-uniform, `off` is the lane's byte offset from `base`.  Non-temporal: every weight
// byte is read once.
__device__ __forceinline__ void dma16(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds), "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void dma4(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2 nt" ::"s"(lds), "v"(off), "s"(base) : "memory");
}
// 32 bytes (eight floats) as two loads into registers
__device__ __forceinline__ void ld_32b(u32x4& lo, u32x4& hi, const LQ4_GLOBAL void* base, uint32_t off) {
    asm volatile("global_load_dwordx4 %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:16"
                 : "=&v"(lo), "=&v"(hi)
                 : "v"(off), "s"(base));
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <typename T>
__device__ __forceinline__ void tie(T& v) {
    asm volatile("" : "+v"(v));
}
// The same loads for a subset of the lanes (`mask`, one bit a lane, not empty): a row's short last slab.
__device__ __forceinline__ void dma16_masked(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off, uint64_t mask) {
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3 nt\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "s"(lds), "v"(off), "s"(base), "s"(mask)
                 : "memory");
}
__device__ __forceinline__ void dma4_masked(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off, uint64_t mask) {
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3 nt\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "s"(lds), "v"(off), "s"(base), "s"(mask)
                 : "memory");
}

// WAVES: waves per workgroup (every workgroup stages the whole activation vector: more waves share one staging on
// longer rows).  XR: 8-activation units a thread stages (K <= 8 * 64 * WAVES * XR).  D: slots in a wave's ring.
// SLABS: 1..3 = rows of exactly that many whole slabs, the lane's blocks of x stay in registers (D is a multiple
// of SLABS, so the slab at an unrolled position is known at compile time); 0 = any row length, x from LDS.
template <int WAVES, int XR, int D, int SLABS>
__global__ __launch_bounds__(WAVES * 64) void gemv_q4_dma(const uint8_t* __restrict__ w_, uint32_t n, uint32_t k,
                                                           const float* __restrict__ x_, float* __restrict__ y) {
    static_assert(SLABS == 0 || D % SLABS == 0, "the slab at an unrolled position must not depend on the round");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds_raw[];
    lds_u32* const xs = (lds_u32*)lds_raw;
    constexpr int T = WAVES * 64;
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t row_bytes = nb * kBlockBytes;
    const uint32_t slabs = SLABS ? SLABS : (nb + 63) / 64;
    const uint32_t last_blocks = nb - (slabs - 1) * 64;  // blocks of a row's last slab
    const uint32_t last_bytes = last_blocks * kBlockBytes;
    const uint32_t wave = uniform(tid >> 6);
    const uint32_t n_waves = gridDim.x * WAVES;
    const uint32_t wid = uniform(blockIdx.x * WAVES + wave);
    const LQ4_GLOBAL uint8_t* const w = as_global(w_);
    const LQ4_GLOBAL float* const x = as_global(x_);
    // the wave's ring: behind the staged activations
    const uint32_t xs_dwords = nb * kXPitch;
    lds_u32* const ring_ptr = xs + xs_dwords + wave * D * (kSlotBytes / 4);
    const uint32_t ring_addr = uniform(static_cast<uint32_t>(reinterpret_cast<size_t>(ring_ptr)));

    // ---- the activations first: requested before any weight so they can be waited for alone ----
    const uint32_t n_units = nb * 4;
    u32x4 xlo[XR], xhi[XR];
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
        ld_32b(xlo[i], xhi[i], x, u * 32u);
    }

    // ---- this wave's rows: one run, the first n % n_waves waves take one row more ----
    const uint32_t share = n / n_waves, extra = n - share * n_waves;
    const uint32_t my_rows = share + (wid < extra ? 1u : 0u);
    const uint32_t first_row = wid * share + (wid < extra ? wid : extra);
    const uint32_t total = my_rows * slabs;  // slots
    // a short last slab: 20 * blocks bytes as whole 16-byte pieces, then the dwords behind them (fewer than four,
    // or what is left past 1024 bytes); lane 0 always takes part in the second load so that it is a load
    // instruction on every path (the waits count them)
    const uint32_t n16 = last_bytes / 16 < 64 ? last_bytes / 16 : 64;
    const uint32_t rest = (last_bytes - n16 * 16) / 4;
    const uint64_t mask16 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < n16);
    const uint64_t mask4 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < (rest ? rest : 1u));
    const bool short_last = SLABS == 0 && last_blocks != 64;

    const LQ4_GLOBAL uint8_t* rq_ptr = w + static_cast<uint64_t>(first_row) * row_bytes;  // the next slot to request
    uint32_t rq_slab = 0;                                                                   // its slab (SLABS == 0)
    const uint32_t off16 = lane * 16u, off4 = lane * 4u;
    auto request_into = [&](uint32_t at) {  // `at`: LDS byte address of the slot
        if (short_last && rq_slab + 1 == slabs) {
            dma16_masked(at, rq_ptr, off16, mask16);
            dma4_masked(at + n16 * 16, rq_ptr + (rest ? n16 * 16 : 0u), off4, mask4);
            rq_ptr += last_bytes;
        } else {
            dma16(at, rq_ptr, off16);
            dma4(at + 1024, rq_ptr + 1024, off4);
            rq_ptr += kSlotBytes;
        }
        if (SLABS == 0) rq_slab = rq_slab + 1 == slabs ? 0 : rq_slab + 1;
    };
    uint32_t to_request = total;
#pragma unroll
    for (int i = 0; i < D; ++i) {
        if (to_request) {  // uniform
            request_into(ring_addr + i * kSlotBytes);
            --to_request;
        }
    }

    // ---- stage x: the activation loads are older than every weight request ----
    if (total >= static_cast<uint32_t>(D)) wait_vm<2 * D>();
    else wait_vm<0>();
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        tie(xlo[i]);
        tie(xhi[i]);
        const bool act = tid + i * T < n_units;
        if (XR == 1 || static_cast<uint32_t>(i * T) < n_units) {
            const u32x4 lo = xlo[i], hi = xhi[i];
            stage_x8(xs, act ? tid + i * T : 0, make_float4(as_f32(lo.x), as_f32(lo.y), as_f32(lo.z), as_f32(lo.w)),
                     make_float4(as_f32(hi.x), as_f32(hi.y), as_f32(hi.z), as_f32(hi.w)), act);
        }
    }
    barrier_lds();

    // ---- the arithmetic: round after round over the ring ----
    constexpr int NX = SLABS ? SLABS : 1;
    XBlock xb[NX];
#pragma unroll
    for (int sl = 0; sl < NX; ++sl) {
        const uint32_t blk = sl * 64 + lane;
        load_xblock(xs, blk < nb ? blk : nb - 1, xb[sl]);
    }
    float acc = 0.0f;
    uint32_t left = total, cs_slab = 0, row = first_row;
    const lds_u32* const my_block = ring_ptr + 5 * lane;  // the lane's block in slot 0: byte 20 l
    while (left) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            if (left == 0) break;  // uniform
            if (to_request) wait_vm<2 * (D - 1)>();  // the ring is full behind the head
            else wait_vm<0>();
            const lds_u32* const slot = my_block + i * (kSlotBytes / 4);
            Q4BlockRaw wb;
            wb.sb = slot[0];
            wb.q[0] = slot[1]; wb.q[1] = slot[2]; wb.q[2] = slot[3]; wb.q[3] = slot[4];
            bool live = true;
            if (SLABS == 0) {
                const uint32_t blk_raw = cs_slab * 64 + lane;
                live = blk_raw < nb;
                if (slabs > 1) load_xblock(xs, live ? blk_raw : nb - 1, xb[0]);
                // a lane past the end of the row has read what the slot held before: scale and bias of zero,
                // whatever bits they were (a stale bias may be an infinity, and zero times that is not zero)
                wb.sb = live ? wb.sb : 0u;
            }
            // The slot is free again once its words are in registers: the empty statement makes the compiler wait
            // for those reads here, ahead of the request that refills the slot.
            asm volatile("" : "+v"(wb.sb), "+v"(wb.q[0]), "+v"(wb.q[1]), "+v"(wb.q[2]), "+v"(wb.q[3]));
            if (to_request) {
                request_into(ring_addr + i * kSlotBytes);
                --to_request;
            }
            acc = block_fma(wb, xb[SLABS ? i % NX : 0], live, acc);
            bool row_done;
            if (SLABS) {
                row_done = i % NX == NX - 1;
            } else {
                row_done = cs_slab + 1 == slabs;
                cs_slab = row_done ? 0 : cs_slab + 1;
            }
            if (row_done) {
                const float v = segment_sum<64>(acc);
                acc = 0.0f;
                if (lane == 63) y[row] = v;
                ++row;
            }
            --left;
        }
    }
    wait_vm<0>();  // nothing of this wave is on its way when it ends
}

struct DmaPlan {
    uint32_t waves, depth, slabs, grid;
    size_t lds;
};

// One entry per instantiation: waves per workgroup, workgroups per CU, ring depth.
bool plan_dma(uint32_t n, uint32_t k, uint32_t cu_count, DmaPlan* out) {
    const uint32_t nb = k / kBlockWeights;
    const size_t xs_bytes = static_cast<size_t>(nb) * kXPitch * 4;
    DmaPlan p;
    if (nb == 64) { p.waves = 4; p.depth = 6; p.slabs = 1; }
    else if (nb == 128) { p.waves = 8; p.depth = 4; p.slabs = 2; }
    else if (nb == 192) { p.waves = 16; p.depth = 6; p.slabs = 3; }
    else if (k <= 2048) { p.waves = 4; p.depth = 4; p.slabs = 0; }
    else if (k <= 8192) { p.waves = 8; p.depth = 4; p.slabs = 0; }
    else if (k <= 24576) { p.waves = 16; p.depth = 3; p.slabs = 0; }
    else return false;
    const uint32_t wg_per_cu = 16 / p.waves;
    p.lds = xs_bytes + static_cast<size_t>(p.waves) * p.depth * kSlotBytes;
    if (p.lds * wg_per_cu > 160 * 1024) return false;
    // every wave resident, rows dealt evenly; fewer workgroups when there are fewer rows than waves
    const uint32_t wgs_resident = cu_count * wg_per_cu;
    const uint32_t wgs_needed = (n + p.waves - 1) / p.waves;
    p.grid = wgs_needed < wgs_resident ? wgs_needed : wgs_resident;
    *out = p;
    return true;
}

template <int WAVES, int XR, int D, int SLABS>
void launch_one(const DmaPlan& p, const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream) {
    static bool attr_set = false;
    if (!attr_set) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_q4_dma<WAVES, XR, D, SLABS>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        attr_set = true;
    }
    hipLaunchKernelGGL((gemv_q4_dma<WAVES, XR, D, SLABS>), dim3(p.grid), dim3(WAVES * 64), p.lds, stream, w, n, k, x, y);
}

}  // namespace

bool gemv_dma_serves(uint32_t n, uint32_t k, uint32_t cu_count) {
    DmaPlan p;
    return n != 0 && plan_dma(n, k, cu_count, &p);
}

void launch_gemv_dma(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, uint32_t cu_count, hipStream_t stream) {
    DmaPlan p;
    if (!plan_dma(n, k, cu_count, &p)) return;  // the caller asked gemv_dma_serves first
    if (p.slabs == 1) launch_one<4, 1, 6, 1>(p, w, n, k, x, y, stream);
    else if (p.slabs == 2) launch_one<8, 2, 4, 2>(p, w, n, k, x, y, stream);
    else if (p.slabs == 3) launch_one<16, 1, 6, 3>(p, w, n, k, x, y, stream);
    else if (p.waves == 4) launch_one<4, 1, 4, 0>(p, w, n, k, x, y, stream);
    else if (p.waves == 8) launch_one<8, 2, 4, 0>(p, w, n, k, x, y, stream);
    else launch_one<16, 3, 3, 0>(p, w, n, k, x, y, stream);
}

}  // namespace lq4
