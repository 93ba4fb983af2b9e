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
// same counter and may complete early, which can only make a wait longer than needed.  The activations take the
// same road (requested ahead of the first weights, so they are waited for alone): each wave brings its 512-element
// piece of x into the staging area as raw floats, reads it back, and after a barrier the pieces are staged over it
// as in the lane-owns-block kernel (lq4_b1_dev.hpp: per-block scaled fixed point, eight-wide 4-bit dot products).
// No load of this kernel has a register as its destination.  That is deliberate: a register which inline assembly
// fills "later" is not safe against the register allocator (a copy it inserts between the load and the wait reads
// the old contents, and it may hand the original register to another value that the arriving data then destroys;
// both happened here, the second as a memory fault through a clobbered address offset).
//
// Work split, rows of more than three slabs (gemv_q4_dma).  A workgroup (one per CU) owns a run of consecutive
// rows, i.e. a run of slots that is also one run of memory, and its sixteen waves cut that run into sixteen equal
// pieces to within one slot, wherever the row boundaries fall: 5120 rows of nine slots are twenty rows a CU, which dealt out as whole rows would leave four
// waves with eighteen slots and twelve with nine.  A wave's slots are again one run of memory, so the address of
// the next request is a running pointer.  A row that starts in one wave and ends in a later one is finished by the
// wave it starts in: every wave leaves the sum of the row that was already under way at its first slot (at most
// one such row) in LDS, and after a barrier the starting wave adds those to its own part in wave order.  The ring has a compile-time depth D and the loop is unrolled D times: the slot a
// wave has just emptied is the one its next request fills, so every LDS offset is a constant, the wait in the
// steady state is the constant vmcnt(2 (D - 1)), and what is left per slot is a dozen scalar instructions.  (A
// first version with run-time ring positions and a wait chosen by a switch spent ~80 scalar instructions and a
// dozen branches per slot and was 10-15 % slower than the lane-owns-block kernel: a CU issues one scalar
// instruction per cycle for all its waves.)  The block of slot s + 1 is read out of LDS before the arithmetic of
// slot s, so that read's latency hides behind ~50 vector instructions, and the refill of slot s is requested after
// them, when its words have long been in registers.  The lane's block of x is read from LDS slot by slot (104 bytes
// a lane: six times the LDS traffic of the weights themselves); rows of up to three slabs, which can keep those
// blocks in registers for the whole launch, have the kernel described at the end.
//
// One workgroup of sixteen waves per CU: the activations are staged once per CU, by as many waves as the vector
// has 512-element pieces (the others skip the staging code altogether, which on short rows is most of what a
// wave of the lane-owns-block kernel executes).
//
// Rows of one to three slabs (gemv_q4_dma_rows: K <= 6144, the lm_heads) are short enough to be handed out whole,
// so there the waves of a workgroup take rows as they come free instead of owning equal pieces: time stamps of the
// equal-pieces form on 248320 x 2048 showed a workgroup's first wave done after 38 us and its last after 48.6, the
// last fifth of the rows streaming from ever fewer waves.  Taking rows from a counter in LDS brings the waves' ends
// within one slot of each other (45.4 / 46.8 us): 248320 x 2048 52.6 -> 51.0 us, 151936 x 5120 80.0 -> 76.2,
// 65536 x 3072 24.7 -> 22.6, 17408 x 5120 13.6 -> 12.3.  A row keeps its ring positions' order (position i holds slab
// i % SLABS), so the blocks of x stay in registers and a row still ends in one cross-lane sum.  Handing out single
// slots of longer rows was tried first and is not kept: the slab a wave meets is then known only at run time, so the
// blocks of x come from LDS for every slot and every slot ends in its own cross-lane sum, which cost more than the
// even ends returned (151936 x 5120 79.5 -> 88.2 us, 32768 x 4096 16.6 -> 17.2, 5120 x 17408 13.4 -> 12.9).  What
// remains uneven is between workgroups (ends 41..52 us in one launch, 44..49 in the next, whole XCDs ahead or behind).
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
// The same for data every workgroup reads (the activations): left to the caches.
__device__ __forceinline__ void dma16_shared(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds), "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void dma4(uint32_t lds, const LQ4_GLOBAL void* base, uint32_t off) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2 nt" ::"s"(lds), "v"(off), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
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

constexpr int kWaves = 16;

// The activations' way into LDS, first half: each wave moves the 512-element pieces it will stage (2 KB of raw floats a
// piece) into the staging area, at the bytes they have in x.  A piece that reaches past the end of x is cut at 16
// bytes (K is a multiple of 32).  Requested before any weight, so that they can be waited for alone.
template <int XR>
__device__ __forceinline__ void request_x(lds_u32* xs, const LQ4_GLOBAL float* x, uint32_t k, uint32_t wave, int lane) {
    constexpr int T = kWaves * 64;
    const uint32_t xs_addr = uniform(static_cast<uint32_t>(reinterpret_cast<size_t>(xs)));
    const uint32_t x_bytes = k * 4;
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const uint32_t piece = (i * T + wave * 64) * 32u;  // first byte
        if (piece < x_bytes) {                           // uniform
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t first = piece + h * 1024u;
                if (first + 1024u <= x_bytes) {
                    dma16_shared(xs_addr + first, x + first / 4, lane * 16u);
                } else if (first < x_bytes) {
                    const uint64_t m = __builtin_amdgcn_ballot_w64(first + lane * 16u < x_bytes);
                    dma16_masked(xs_addr + first, x + first / 4, lane * 16u, m);
                }
            }
        }
    }
}

// Second half, once the wave's own pieces have landed (the caller has waited for them): the raw floats out of the
// staging area, a barrier, the staged form (lq4_b1_dev.hpp) over them, a barrier.
template <int XR>
__device__ __forceinline__ void stage_x(lds_u32* xs, uint32_t k, uint32_t wave, int tid) {
    constexpr int T = kWaves * 64;
    const uint32_t n_units = k / 8, x_bytes = k * 4;
    float4 xa[XR], xc[XR];
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        xa[i] = xc[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if ((i * T + wave * 64) * 32u < x_bytes) {  // uniform: this wave's own piece
            const uint32_t u = tid + i * T < n_units ? tid + i * T : 0;
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const LQ4_LDS f32x4* const raw = reinterpret_cast<const LQ4_LDS f32x4*>(xs + u * 8);
            const f32x4 lo = raw[0], hi = raw[1];
            xa[i] = make_float4(lo.x, lo.y, lo.z, lo.w);
            xc[i] = make_float4(hi.x, hi.y, hi.z, hi.w);
        }
    }
    barrier_lds();  // every piece has been read: the staged form may overwrite the raw one
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        if ((i * T + wave * 64) * 32u < x_bytes) {  // uniform
            const bool act = tid + i * T < n_units;
            stage_x8(xs, act ? tid + i * T : 0, xa[i], xc[i], act);
        }
    }
    barrier_lds();
}

// Rows of any length (launched for more than three slabs; up to three have the kernel below): the lane's block of x
// comes from LDS for every slot.  XR: 8-activation units a thread stages (K <= 8 * 1024 * XR).  D: slots in a wave's
// ring.
template <int XR, int D>
__global__ __launch_bounds__(kWaves * 64) void gemv_q4_dma(const uint8_t* __restrict__ w_, uint32_t n, uint32_t k,
                                                            const float* __restrict__ x_, float* __restrict__ y) {
    static_assert(D >= 3, "one slot in registers, one landed, at least one on its way");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds_raw[];
    lds_u32* const xs = (lds_u32*)lds_raw;
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t nb = k / kBlockWeights;
    const uint32_t row_bytes = nb * kBlockBytes;
    const uint32_t slabs = (nb + 63) / 64;
    const uint32_t last_blocks = nb - (slabs - 1) * 64;  // blocks of a row's last slab
    const uint32_t last_bytes = last_blocks * kBlockBytes;
    const uint32_t wave = uniform(tid >> 6);
    const LQ4_GLOBAL uint8_t* const w = as_global(w_);
    const LQ4_GLOBAL float* const x = as_global(x_);
    // LDS: the staged activations | one partial sum a wave | the waves' rings
    const uint32_t xs_dwords = nb * kXPitch;
    LQ4_LDS float* const part = reinterpret_cast<LQ4_LDS float*>(xs + xs_dwords);
    lds_u32* const ring_ptr = xs + xs_dwords + kWaves + wave * D * (kSlotBytes / 4);
    const uint32_t ring_addr = uniform(static_cast<uint32_t>(reinterpret_cast<size_t>(ring_ptr)));

    // ---- the activations first: requested before any weight so they can be waited for alone ----
    request_x<XR>(xs, x, k, wave, lane);

    // ---- this wave's slots ----
    // the workgroup's rows: one run, the first n % workgroups of them take one row more
    const uint32_t share = n / gridDim.x, extra = n - share * gridDim.x;
    const uint32_t wg_rows = share + (blockIdx.x < extra ? 1u : 0u);
    const uint32_t wg_first = blockIdx.x * share + (blockIdx.x < extra ? blockIdx.x : extra);
    const uint32_t wg_slots = wg_rows * slabs;
    auto piece_start = [&](uint32_t j) { return static_cast<uint32_t>(static_cast<uint64_t>(j) * wg_slots / kWaves); };
    const uint32_t s0 = uniform(piece_start(wave)), s1 = uniform(piece_start(wave + 1));
    const uint32_t total = s1 - s0;
    const uint32_t row0 = uniform(s0 / slabs), slab0 = s0 - row0 * slabs;  // where the first slot lies
    // a short last slab: 20 * blocks bytes as whole 16-byte pieces, then the dwords behind them (fewer than four,
    // or what is left past 1024 bytes); lane 0 always takes part in the second load so that it is a load
    // instruction on every path (the waits count them)
    const uint32_t n16 = last_bytes / 16 < 64 ? last_bytes / 16 : 64;
    const uint32_t rest = (last_bytes - n16 * 16) / 4;
    const uint64_t mask16 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < n16);
    const uint64_t mask4 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < (rest ? rest : 1u));
    const bool short_last = last_blocks != 64;

    // the next slot to request: its address and its slab
    const LQ4_GLOBAL uint8_t* rq_ptr = w + static_cast<uint64_t>(wg_first + row0) * row_bytes + slab0 * static_cast<uint32_t>(kSlotBytes);
    uint32_t rq_slab = slab0;
    const uint32_t off16 = lane * 16u, off4 = lane * 4u;
    auto request_next = [&](int pos) {  // `pos`: ring position
        const uint32_t at = ring_addr + pos * kSlotBytes;
        const bool last = rq_slab + 1 == slabs;
        if (short_last && last) {
            dma16_masked(at, rq_ptr, off16, mask16);
            dma4_masked(at + n16 * 16, rq_ptr + (rest ? n16 * 16 : 0u), off4, mask4);
            rq_ptr += last_bytes;
        } else {
            dma16(at, rq_ptr, off16);
            dma4(at + 1024, rq_ptr + 1024, off4);
            rq_ptr += kSlotBytes;
        }
        rq_slab = last ? 0 : rq_slab + 1;
    };
    // Two slots a wave now, the rest of the ring once the activations are staged: a CU accepts requests only as fast
    // as earlier ones are answered once a few dozen KB are on their way, and a wave stuck issuing its whole ring
    // would reach the staging barriers only when most of that data has arrived.
    constexpr int E = 2;
    uint32_t to_request = total;
#pragma unroll
    for (int i = 0; i < E; ++i) {
        if (to_request) {  // uniform
            request_next(i);
            --to_request;
        }
    }

    // ---- stage x: the activation loads are older than every weight request ----
    if (total >= static_cast<uint32_t>(E)) wait_vm<2 * E>();
    else wait_vm<0>();
    stage_x<XR>(xs, k, wave, tid);
#pragma unroll
    for (int i = E; i < D; ++i) {
        if (to_request) {  // uniform
            request_next(i);
            --to_request;
        }
    }

    // ---- the arithmetic: round after round over the ring ----
    XBlock xb;
    const lds_u32* const my_block = ring_ptr + 5 * lane;  // the lane's block in position 0: byte 20 l
    auto read_block = [&](int pos, Q4BlockRaw& wb) {
        const lds_u32* const slot = my_block + pos * (kSlotBytes / 4);
        wb.sb = slot[0];
        wb.q[0] = slot[1]; wb.q[1] = slot[2]; wb.q[2] = slot[3]; wb.q[3] = slot[4];
    };
    float acc = 0.0f;
    uint32_t left = total, cs_slab = slab0, row = wg_first + row0;
    bool in_head = slab0 != 0;  // the row under way at the first slot started in an earlier wave
    Q4BlockRaw cur, nxt;
    if (left) {
        if (total >= static_cast<uint32_t>(D)) wait_vm<2 * (D - 1)>();
        else wait_vm<0>();
        read_block(0, cur);
    }
    while (left) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            if (left == 0) break;  // uniform
            // the slot behind this one out of LDS now: its read hides behind this slot's arithmetic
            if (left > 1) {
                if (to_request) wait_vm<2 * (D - 2)>();  // the ring is full behind this slot
                else wait_vm<0>();
                read_block((i + 1) % D, nxt);
            }
            const bool last_slab = cs_slab + 1 == slabs;
            const uint32_t blk_raw = cs_slab * 64 + lane;
            const bool live = blk_raw < nb;
            load_xblock(xs, live ? blk_raw : nb - 1, xb);
            cs_slab = last_slab ? 0 : cs_slab + 1;
            // a lane past the end of the row has read what the slot held before: scale and bias of zero,
            // whatever bits they were (a stale bias may be an infinity, and zero times that is not zero)
            if (short_last && last_slab) cur.sb = live ? cur.sb : 0u;
            acc = block_fma(cur, xb, live, acc);
            // the slot's words went into registers a slot ago: its place in the ring can be filled again
            if (to_request) {
                request_next(i);
                --to_request;
            }
            if (last_slab) {
                const float v = segment_sum<64>(acc);
                acc = 0.0f;
                if (in_head) {  // uniform: the tail of a row that an earlier wave finishes
                    if (lane == 63) part[wave] = v;
                    in_head = false;
                } else if (lane == 63) {
                    y[row] = v;
                }
                ++row;
            }
            cur = nxt;
            --left;
        }
    }
    wait_vm<0>();  // nothing of this wave is on its way when it ends
    // ---- rows that straddle waves ----
    const bool open_row = total != 0 && cs_slab != 0;  // the last slot did not end its row
    float own = 0.0f;
    if (open_row) {
        own = segment_sum<64>(acc);
        if (in_head && lane == 63) part[wave] = own;  // the whole piece lies inside a row begun earlier
    }
    barrier_lds();
    if (open_row && !in_head) {
        // this wave began the row: the pieces behind it, in wave order, until the one that ends the row
        const uint32_t row_end = (row - wg_first + 1) * slabs;  // first slot of the next row
        for (uint32_t j = wave + 1; j < static_cast<uint32_t>(kWaves); ++j) {
            const uint32_t b = piece_start(j), e = piece_start(j + 1);
            if (b >= row_end) break;
            if (e > b) own += part[j];
        }
        if (lane == 63) y[row] = own;
    }
}

// Rows of one to three slabs (K <= 6144): the lane's blocks of x stay in registers and a wave works on whole rows.
// The waves of a workgroup do not advance at one pace (with equal shares the first is done
// when the last has a fifth of its rows to go, and what is left then streams from fewer waves), so only a wave's
// first D / SLABS rows are fixed: row 16 j + wave goes into ring positions SLABS j .., the sixteen waves' requests
// forming one run of memory, and every later row is the next one nobody has asked for yet, from a counter in LDS:
// taken when the first slab of the row it replaces has been consumed, its slabs requested one by one as their
// positions come free.  Position i of the ring always holds slab i % SLABS (D is a multiple of SLABS), so every
// register index and LDS offset of the unrolled loop is a constant.
template <int D, int SLABS>
__global__ __launch_bounds__(kWaves * 64) void gemv_q4_dma_rows(const uint8_t* __restrict__ w_, uint32_t n, uint32_t k,
                                                                 const float* __restrict__ x_, float* __restrict__ y) {
    static_assert(D >= 3 && SLABS >= 1 && SLABS <= 3 && D % SLABS == 0, "whole rows in the ring");
    extern __shared__ __attribute__((aligned(16))) uint32_t lds_raw[];
    lds_u32* const xs = (lds_u32*)lds_raw;
    const int tid = threadIdx.x, lane = tid & 63;
    const uint32_t nb = k / kBlockWeights;  // at most 64 SLABS, more than 64 (SLABS - 1)
    const uint32_t row_bytes = nb * kBlockBytes;
    const uint32_t last_blocks = nb - (SLABS - 1) * 64;  // blocks of a row's last slab
    const uint32_t last_bytes = last_blocks * kBlockBytes;
    const uint32_t wave = uniform(tid >> 6);
    const LQ4_GLOBAL uint8_t* const w = as_global(w_);
    // LDS: the staged activations | the row counter | the waves' rings
    const uint32_t xs_dwords = nb * kXPitch;
    lds_u32* const counter = xs + xs_dwords;
    lds_u32* const ring_ptr = counter + kWaves + wave * D * (kSlotBytes / 4);
    const uint32_t ring_addr = uniform(static_cast<uint32_t>(reinterpret_cast<size_t>(ring_ptr)));

    request_x<1>(xs, as_global(x_), k, wave, lane);

    // the workgroup's rows: one run, the first n % workgroups of them take one row more
    const uint32_t share = n / gridDim.x, extra = n - share * gridDim.x;
    const uint32_t wg_rows = share + (blockIdx.x < extra ? 1u : 0u);
    const uint32_t wg_first = blockIdx.x * share + (blockIdx.x < extra ? blockIdx.x : extra);
    // a short last slab: 20 * blocks bytes as whole 16-byte pieces, then the dwords behind them (fewer than four, or
    // what is left past 1024 bytes); lane 0 always takes part in the second load so that it is a load instruction on
    // every path (the waits count them)
    const uint32_t n16 = last_bytes / 16 < 64 ? last_bytes / 16 : 64;
    const uint32_t rest = (last_bytes - n16 * 16) / 4;
    const uint64_t mask16 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < n16);
    const uint64_t mask4 = __builtin_amdgcn_ballot_w64(static_cast<uint32_t>(lane) < (rest ? rest : 1u));
    const bool short_last = last_blocks != 64;
    const LQ4_GLOBAL uint8_t* const w_wg = w + static_cast<uint64_t>(wg_first) * row_bytes;
    const uint32_t off16 = lane * 16u, off4 = lane * 4u;
    uint32_t slot_row[D];  // the row in each ring position (scalar registers: the positions are constants)
    auto request = [&](int pos, uint32_t row) {  // slab pos % SLABS of row `row` of the workgroup into ring position `pos`
        const int slab = pos % SLABS;
        const LQ4_GLOBAL uint8_t* const src = w_wg + static_cast<uint64_t>(row) * row_bytes + slab * kSlotBytes;
        const uint32_t at = ring_addr + pos * kSlotBytes;
        if (short_last && slab == SLABS - 1) {
            dma16_masked(at, src, off16, mask16);
            dma4_masked(at + n16 * 16, src + (rest ? n16 * 16 : 0u), off4, mask4);
        } else {
            dma16(at, src, off16);
            dma4(at + 1024, src + 1024, off4);
        }
        slot_row[pos] = row;
    };
    // two slots a wave now, the rest of the ring once the activations are staged (as in the kernel above)
    constexpr int E = 2;
    uint32_t have = 0;  // occupied ring positions: always consecutive ones
#pragma unroll
    for (int i = 0; i < E; ++i) {
        const uint32_t row = (i / SLABS) * kWaves + wave;
        if (row < wg_rows) {  // uniform
            request(i, row);
            ++have;
        }
    }
    if (tid == 0) *counter = (D / SLABS) * kWaves;  // the first row that is nobody's yet

    // ---- stage x: the activation loads are older than every weight request ----
    if (have == static_cast<uint32_t>(E)) wait_vm<2 * E>();
    else wait_vm<0>();
    stage_x<1>(xs, k, wave, tid);  // (its barriers publish the counter as well)
#pragma unroll
    for (int i = E; i < D; ++i) {
        const uint32_t row = (i / SLABS) * kWaves + wave;
        if (row < wg_rows) {  // uniform
            request(i, row);
            ++have;
        }
    }
    // a wave that found fewer than D / SLABS rows finds none behind them either; from the first request the counter
    // turns down on, a wave asks no more: its occupied positions stay consecutive and the ring drains
    bool more = have == static_cast<uint32_t>(D);

    // ---- the arithmetic: round after round over the ring ----
    XBlock xb[SLABS];
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl) {
        const uint32_t blk = sl * 64 + lane;
        load_xblock(xs, blk < nb ? blk : nb - 1, xb[sl]);
    }
    const bool live_last = static_cast<uint32_t>(lane) < last_blocks;
    const lds_u32* const my_block = ring_ptr + 5 * lane;  // the lane's block in position 0: byte 20 l
    auto read_block = [&](int pos, Q4BlockRaw& wb) {
        const lds_u32* const slot = my_block + pos * (kSlotBytes / 4);
        wb.sb = slot[0];
        wb.q[0] = slot[1]; wb.q[1] = slot[2]; wb.q[2] = slot[3]; wb.q[3] = slot[4];
    };
    Q4BlockRaw cur, nxt;
    float acc = 0.0f;
    uint32_t next_row = 0;  // the row whose slabs are replacing the row under way (while `more`)
    if (have) {
        if (more) wait_vm<2 * (D - 1)>();
        else wait_vm<0>();
        read_block(0, cur);
    }
    while (have) {
#pragma unroll
        for (int i = 0; i < D; ++i) {
            if (have == 0) break;  // uniform
            const int slab = i % SLABS;  // a constant once the loop is unrolled
            // at a row's first slab: the row that will take this row's positions, asked for now, needed after the
            // arithmetic.  (A plain LDS atomic of one lane; the wave-wide ds_append was tried for it and did not
            // count as its description says.)
            uint32_t claim = 0;
            if (slab == 0 && more && lane == 0)
                claim = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            // the slot behind this one out of LDS now: its read hides behind this slot's arithmetic
            if (have > 1) {
                if (more) wait_vm<2 * (D - 2)>();  // the ring is full behind this slot
                else wait_vm<0>();
                read_block((i + 1) % D, nxt);
            }
            // a lane past the end of the row has read what the slot held before: scale and bias of zero,
            // whatever bits they were (a stale bias may be an infinity, and zero times that is not zero)
            const bool live = slab == SLABS - 1 ? live_last : true;
            if (short_last && slab == SLABS - 1) cur.sb = live ? cur.sb : 0u;
            acc = block_fma(cur, xb[slab], live, acc);
            if (slab == SLABS - 1) {
                const float v = segment_sum<64>(acc);
                acc = 0.0f;
                if (lane == 63) y[wg_first + slot_row[i]] = v;
            }
            // the slot's words went into registers a slot ago: its place in the ring can be filled again
            if (more) {
                if (slab == 0) {
                    next_row = uniform(claim);
                    if (next_row >= wg_rows) more = false;
                }
            }
            if (more) request(i, next_row);
            else --have;
            cur = nxt;
        }
    }
    wait_vm<0>();  // nothing of this wave is on its way when it ends
}

struct DmaPlan {
    uint32_t xr, depth, slabs, grid;
    size_t lds;
};

// Which instantiation serves a row length (ring depth: see launch_gemv_dma).
bool plan_dma(uint32_t n, uint32_t k, uint32_t cu_count, DmaPlan* out) {
    const uint32_t nb = k / kBlockWeights;
    // (sixteen dwords between the activations and the rings: the waves' partial sums, or the row counter)
    const size_t fixed = static_cast<size_t>(nb) * kXPitch * 4 + kWaves * 4;
    DmaPlan p;
    p.slabs = nb <= 192 ? (nb + 63) / 64 : 0;
    p.xr = k <= 8192 ? 1 : 3;
    p.depth = p.slabs == 2 ? 4 : 3;
    p.lds = fixed + static_cast<size_t>(kWaves) * p.depth * kSlotBytes;
    if (k > 24576 || p.lds > 160 * 1024) return false;
    // one workgroup per CU, rows dealt evenly; fewer workgroups when there are fewer rows than CUs
    p.grid = n < cu_count ? n : cu_count;
    *out = p;
    return true;
}

template <int D, int SLABS>
void launch_rows(const DmaPlan& p, const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q4_dma_rows<D, SLABS>), 160 * 1024);
    const size_t lds = p.lds < 96 * 1024 ? 96 * 1024 : p.lds;  // one workgroup to a CU
    hipLaunchKernelGGL((gemv_q4_dma_rows<D, SLABS>), dim3(p.grid), dim3(kWaves * 64), lds, stream, w, n, k, x, y);
}

template <int XR, int D>
void launch_one(const DmaPlan& p, const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream) {
    static LdsCapOnce lds_cap;
    lds_cap.raise(reinterpret_cast<const void*>(gemv_q4_dma<XR, D>), 160 * 1024);
    // at least half a CU's LDS, so that the workgroups spread one to a CU
    const size_t lds = p.lds < 96 * 1024 ? 96 * 1024 : p.lds;
    hipLaunchKernelGGL((gemv_q4_dma<XR, D>), dim3(p.grid), dim3(kWaves * 64), lds, stream, w, n, k, x, y);
}

}  // namespace

bool gemv_dma_serves(uint32_t n, uint32_t k, uint32_t cu_count) {
    DmaPlan p;
    return n != 0 && plan_dma(n, k, cu_count, &p);
}

// Measured against the lane-owns-block kernel on 256 CUs (us, that kernel -> this one, ring depth three):
//   large: 248320 x 2048 62.1 -> 49.6; 151936 x 5120 87.8 -> 75.1; 65536 x 2048 (84 MB) 17.4 -> 15.3; 17408 x 5120 (56 MB)
//     12.6 -> 11.6; 32768 x 2048 (42 MB) 10.2 -> 9.1; 16384 x 4096 9.6 -> 9.2; 8192 x 8192 10.7 -> 9.7; 12288 x 5120 (39 MB)
//     10.3 -> 9.4; 4096 x 14336 (37 MB) 10.8 -> 9.4; 8192 x 6144 (31 MB) 8.4 -> 7.9; 20480 x 2048 (26 MB) 7.2 -> 6.9;
//     5120 x 17408 16.8 -> 13.5; 3072 x 12288 (24 MB) 9.3 -> 8.2; level at 16384 x 2048 (21 MB, 6.1) and 12288 x 2048 (16 MB,
//     5.2); behind with few long rows (2048 x 17408, 22 MB: 8.6 -> 9.1);
//   rows that are not whole 2048-weight slabs, where the other kernel's lanes idle through part of a step: 24576 x
//     2560 12.9 -> 9.7; 12288 x 3072 8.9 -> 6.7; 9728 x 2560 (16 MB) 8.3 -> 5.9; 8192 x 3072 7.5 -> 5.5; 6144 x 3584 6.5 -> 4.9;
//     6144 x 2560 (10 MB) 6.1 -> 4.6; 4096 x 3072 (8 MB) 6.0 -> 4.0; 6144 x 5120 7.5 -> 6.4;
//   rows of two slabs: 6144 x 4096 (16 MB) 6.1 -> 5.0; 8192 x 4096 6.4 -> 6.1;
//   level or behind below that: 4096 x 8192 6.8 -> 6.9, 4096 x 6144 5.5 -> 5.7, 2048 x 6144 (8 MB) 3.7 -> 4.7, every row
//     shorter than one slab (131072 x 1024 18.9 -> 21.7: the other kernel puts two rows side by side in a wave) and the
//     decode layer's matrices (its start costs two workgroup barriers of sixteen waves).
bool gemv_dma_pays(uint32_t n, uint32_t k, uint32_t cu_count) {
    if (!gemv_dma_serves(n, k, cu_count) || k < 2048) return false;
    const uint64_t bytes = static_cast<uint64_t>(n) * (k / kBlockWeights) * kBlockBytes;
    if (bytes >= (20ull << 20) && n >= 3072) return true;
    if (k % 2048 != 0) return bytes >= (6ull << 20);
    return k == 4096 && bytes >= (12ull << 20);
}

void launch_gemv_dma(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, uint32_t cu_count, hipStream_t stream) {
    DmaPlan p;
    if (!plan_dma(n, k, cu_count, &p)) return;  // the caller asked gemv_dma_serves first
    // Ring depth: the least the kernels allow (three slots a wave; four where a row is two slabs).  Six were measured
    // slower on every shape (248320 x 2048 51.4 -> 49.6 us, 17408 x 5120 12.3 -> 11.6, 151936 x 5120 76.3 -> 75.1,
    // 65536 x 2048 16.4 -> 15.3, 32768 x 4096 16.0 -> 14.9, 16384 x 8192 18.0 -> 16.1, 32768 x 3072 13.5 -> 12.4): what a
    // CU has asked for beyond its share of the memory system only queues.
    if (p.slabs == 1) launch_rows<3, 1>(p, w, n, k, x, y, stream);
    else if (p.slabs == 2) launch_rows<4, 2>(p, w, n, k, x, y, stream);
    else if (p.slabs == 3) launch_rows<3, 3>(p, w, n, k, x, y, stream);
    else if (p.xr == 1) launch_one<1, 3>(p, w, n, k, x, y, stream);
    else launch_one<3, 3>(p, w, n, k, x, y, stream);
}

}  // namespace lq4
