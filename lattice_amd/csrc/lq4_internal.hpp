// Internal declarations shared by the translation units of liblattice_hip_q4.so.
// Kernel launchers validate nothing: the C ABI layer (lq4_api.hip) checks every
// shape, alignment and bound before a launcher is called.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace lq4 {

// A kernel's dynamic-LDS cap (hipFuncAttributeMaxDynamicSharedMemorySize) belongs to one device's copy of the code,
// so a launcher raises it once on every device it launches on: one bit a device, one object (static, in the
// launcher) per kernel instantiation.  Two threads that race both set the attribute, which is harmless.
struct LdsCapOnce {
    std::atomic<uint64_t> done{0};
    void raise(const void* kernel, int bytes) {
        int dev = 0;
        (void)hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (done.load(std::memory_order_relaxed) & bit) return;
        (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        done.fetch_or(bit, std::memory_order_relaxed);
    }
};

constexpr int kBlockBytes = 20;    // one Q4 block: u16 scale, u16 bias, 16 packed bytes
constexpr int kBlockWeights = 32;  // weights per block
constexpr int kMaxLoraRank = 64;
constexpr int kMaxGemvBatch = 16;

// Optional LoRA epilogue operands.  t = A.x is produced by launch_lora_a into
// ctx scratch before the main kernel runs (or, for one token, inside the main kernel's
// launch: see `a` below); the main kernel adds
// scale * sum_j B[n,j] * t[row,j] before its single store of y.
struct LoraEpilogue {
    const void* b;     // [d_out, rank] row-major, f32 or f16
    const float* t;    // [rows, rank] f32
    uint32_t rank;     // 0 = no LoRA
    int b_is_f16;
    float scale;
    // Batch-1 GEMV only.  With `a` set the launch carries `rank` extra workgroups that compute
    // t = A.x themselves while the others stream weights, so no separate launch precedes it.
    // Producer j stores slots[j] = {bits of t[j], tag of the launch} as one 64-bit word; the tag is the place of
    // the launch's dispatch packet in its queue, which every workgroup of the launch reads from its own input
    // registers, so nothing has to be agreed on through memory and nothing has to be reset between launches.  A
    // weight wave polls the slots until all carry its tag (at most `spin_limit` polls, then it computes t on its
    // own and counts itself in sync[2]).
    const void* a;     // [rank, d_in] row-major, f32 or f16 (b_is_f16 applies to both factors); the few-token GEMM
                       // takes its packed A here (see gemm_skinny_pack_lora_a)
    unsigned long long* slots;  // [kMaxLoraRank]
    uint32_t* sync;
    uint32_t spin_limit;
};

// Several matrices with rows of the same K against one activation vector in one batch-1 launch: the rows of the
// views stacked one under the other, view v = rows [begin[v], begin[v + 1]).  Each view has its own output and its
// own LoRA epilogue (rank 0 = none; t = A . x is in memory when the launch starts).
constexpr int kMaxViews = 8;
struct MultiViews {
    uint32_t count;
    uint32_t begin[kMaxViews + 1];
    const uint8_t* w[kMaxViews];
    float* y[kMaxViews];
    const void* b[kMaxViews];   // [n_v, rank] row-major, f32 or f16
    const float* t[kMaxViews];  // [rank] f32
    uint32_t rank[kMaxViews];
    int b_is_f16[kMaxViews];
    float scale[kMaxViews];
    // when the launch computes the factors itself (the LoraEpilogue beside it then carries the hand-over words and
    // rank = the ranks' sum, at most 64): the A matrices, and where each view's factors start in the stacked t
    const void* a[kMaxViews];   // [rank, k] row-major, dtype as b
    uint32_t t_off[kMaxViews];
};

// The A factors of the views' adapters for one launch that computes every t_v = A_v . x (rank 0 = no adapter).
struct LoraAViews {
    uint32_t count;
    const void* a[kMaxViews];  // [rank, d_in] row-major, f32 or f16
    float* t[kMaxViews];       // [rows, rank] f32
    uint32_t rank[kMaxViews];
    int a_is_f16[kMaxViews];
};
bool gemv_multi_serves(const MultiViews& mv, uint32_t k);
// The same for 2..8 activation rows on the integer matrix-core kernel (views of whole 16-row tiles; t in memory).
bool gemv_i8_multi_serves(const MultiViews& mv, uint32_t k, uint32_t batch, uint32_t cu_count);
void launch_gemv_i8_multi(const MultiViews& mv, uint32_t k, const float* x, uint32_t x_stride, uint32_t batch,
                          uint32_t cu_count, const LoraEpilogue* in_launch, hipStream_t stream);
// `in_launch`: null = every t_v is in memory; else the hand-over words (slots, sync, spin_limit, rank = the ranks' sum)
// of a launch that computes the factors in producer workgroups of its own.
void launch_gemv_multi(const MultiViews& mv, uint32_t k, const float* x, const LoraEpilogue* in_launch, hipStream_t stream);
void launch_lora_a_views(const LoraAViews& av, uint32_t d_in, const float* x, uint32_t x_stride, uint32_t rows,
                         hipStream_t stream);

// Elementwise steps fused into the batch-1 GEMV.
//   prologue kAddNorm: v = base + delta (delta may be null), the activation is the shifted RMSNorm
//     v * rsqrt(mean(v^2) + eps) * (1 + gamma); workgroup 0 also writes v to residual_out if set
//     (residual_out must not alias base or delta: other workgroups still read them).
//   prologue kSiluMul: x holds [gate(K) | up(K)], the activation is silu(gate) * up.
//   epilogue kAddResidual: residual[n] += y[n]; copy_dst[n] = residual[n] if set; y itself is
//     stored only if its pointer is not null.
struct GemvFusion {
    enum Prologue : int { kPlain = 0, kAddNorm = 1, kSiluMul = 2 };
    // kSiluMulPairs: W = [n / 2 gate rows | n / 2 up rows], y[i] = silu(W_i . x) * (W_(n/2 + i) . x), i < n / 2
    // (the batch-1 kernel at rows of 2048 weights and more, without LoRA; see gemv_b1_pairs_served)
    enum Epilogue : int { kStore = 0, kAddResidual = 1, kSiluMulPairs = 2 };
    int prologue;
    const float* base;
    const float* delta;
    const float* gamma;
    float eps;
    float* residual_out;
    int epilogue;
    float* residual;
    float* copy_dst;
};

// y[b, n] = W . x[b]  (+ LoRA), b < batch <= kMaxGemvBatch.  x rows are `x_stride`
// floats apart, y rows `y_stride` floats apart.
void launch_gemv(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride,
                 uint32_t batch, float* y, uint32_t y_stride, const LoraEpilogue& lora,
                 hipStream_t stream);

// Batch-1 fast path (x staged in LDS as per-block fixed point, lq4_b1_dev.hpp); needs gemv_b1_lds_bytes(k) of LDS.
size_t gemv_b1_lds_bytes(uint32_t k);
bool gemv_b1_pairs_served(uint32_t n, uint32_t k);
void launch_gemv_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y,
                    const LoraEpilogue& lora, hipStream_t stream);
// 2..8 activation rows on the integer matrix cores (lq4_gemv_i8.hip): y = W . x, optional LoRA epilogue with t in
// memory or computed by producer workgroups of the launch (gemv_i8_lora_in_launch).  gemv_i8_serves: the staged activations fit the LDS (K up to about 7000).
// Tall matrices of short rows (at least two 16-row tiles per CU, K up to about 2900), which the kernel serves with
// two eight-wave workgroups per CU.
bool gemv_i8_many_short_rows(uint32_t n, uint32_t k, uint32_t cu_count);
bool gemv_i8_serves(uint32_t n, uint32_t k, uint32_t batch, uint32_t cu_count);
// true = the launch has room for `rank_total` producer workgroups that compute the LoRA factors t = A . x themselves
// (LoraEpilogue::a and ::slots set, [rank_total][8] slots; for several views a, t_off of MultiViews and
// in_launch->rank = rank_total): no launch for t has to precede.
bool gemv_i8_lora_in_launch(uint32_t n, uint32_t k, uint32_t batch, uint32_t rank_total, uint32_t cu_count);
void launch_gemv_i8(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride, uint32_t batch,
                    float* y, uint32_t y_stride, const LoraEpilogue& lora, uint32_t cu_count, hipStream_t stream);

// Batch-1 kernel whose weights go from memory straight into a per-wave ring of LDS slots (lq4_gemv_dma.hip): plain
// y = W . x only.  gemv_dma_serves: the shape fits (K <= 24576 and LDS for the activations plus two slots a wave).
bool gemv_dma_serves(uint32_t n, uint32_t k, uint32_t cu_count);
// ... and it is measured faster than the lane-owns-block kernel there (full slabs, enough bytes to hide its start).
bool gemv_dma_pays(uint32_t n, uint32_t k, uint32_t cu_count);
void launch_gemv_dma(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, uint32_t cu_count, hipStream_t stream);
// Same with fused elementwise steps (separate kernel instantiations; the plain ones are untouched).
void launch_gemv_b1_fused(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y,
                          const LoraEpilogue& lora, const GemvFusion& fusion, hipStream_t stream);

// Stand-alone forms of the same steps for any number of rows.
//   residual_add_norm: v = base + delta (delta may be null); residual_out = v if set;
//     normed_out = shifted RMSNorm of v.  Rows are `hidden` floats apart.
//   silu_mul: out[r, i] = silu(gu[r, i]) * gu[r, count + i]; out rows out_stride floats apart
//     (out == gate_up with out_stride == 2 * count is the in-place form).
//   add_and_copy: residual += src; dst = residual if set.
void launch_residual_add_norm(const float* base, const float* delta, const float* gamma, uint32_t hidden,
                              uint32_t rows, float eps, float* residual_out, float* normed_out, hipStream_t stream);
void launch_silu_mul(const float* gate_up, uint32_t count, uint32_t rows, float* out, uint32_t out_stride,
                     hipStream_t stream);
void launch_add_and_copy(const float* src, float* residual, float* dst, size_t count, hipStream_t stream);
// Routed experts for a few tokens as per-pair one-token GEMVs (lq4_moe_b1.hip): gate||up into scratch
// (moe_b1_scratch_bytes), then down with silu, the routing weights and the sum over the slots inside it.
// `slots` = top_k, or top_k + 1 with the shared expert riding along (its tensors and gate vector given,
// its intermediate size equal to `inter`).  Serves hidden <= 8192 and slots * inter <= 8192.  With
// `route_logits` [tokens, E] (E <= 256) the gate||up launch routes itself and stores ids and weights to
// ids_out / wts_out (`ids` / `weights` are then ignored).  top_k == 0 with the shared tensors is the shared
// expert alone; `accumulate` then adds it onto y (the routed experts' sum) instead of overwriting y.
bool moe_b1_serves(uint32_t inter, uint32_t hidden, uint32_t slots);
size_t moe_b1_scratch_bytes(uint32_t tokens, uint32_t slots, uint32_t inter);
void launch_moe_b1(const uint8_t* gate_up, const uint8_t* down, uint32_t num_experts, uint32_t inter, uint32_t hidden,
                   const float* x, uint32_t tokens, const int32_t* ids, const float* weights, uint32_t top_k, float* y,
                   float* scratch, const uint8_t* shared_gate_up, const uint8_t* shared_down, const float* shared_gate,
                   const float* route_logits, int32_t* ids_out, float* wts_out, bool accumulate, hipStream_t stream);
// y[t, :] = fma(sigmoid(x[t] . gate), shared_out[t, :], y[t, :]) for every token
void launch_moe_shared_gate_add(const float* x, const float* gate, const float* shared_out, uint32_t hidden,
                                uint32_t tokens, float* y, hipStream_t stream);

// Matrix-core GEMV for batch 1..8 (activations staged in LDS as f16 columns).
size_t gemv_mfma_lds_bytes(uint32_t k, uint32_t batch);
void launch_gemv_mfma(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t x_stride,
                      uint32_t batch, float* y, uint32_t y_stride, const LoraEpilogue& lora,
                      hipStream_t stream, const GemvFusion* fusion = nullptr);
// The batch form of launch_gemv_b1_fused for 2..kMaxGemvBatch activation rows: base, delta and
// residual_out are [batch, K], x for kSiluMul is [batch, 2K] ([gate | up] per row), y, residual and
// copy_dst are [batch, N].  False (nothing launched) when the staged rows do not fit in LDS.
bool gemv_fused_batch_fits(uint32_t k, uint32_t batch);
bool launch_gemv_fused_batch(const uint8_t* w, uint32_t n, uint32_t k, const float* x, uint32_t batch, float* y,
                             const GemvFusion& fusion, hipStream_t stream);

// t[row, j] = sum_k A[j, k] * x[row, k]; x f32 or f16 with row stride x_stride elements.
void launch_lora_a(const void* a, int a_is_f16, uint32_t rank, uint32_t d_in, const void* x,
                   int x_is_f16, uint32_t x_stride, uint32_t rows, float* t, hipStream_t stream);

// y[row, n] += scale * sum_j B[n, j] * t[row, j]  for row < rows.
void launch_lora_b_accum(const void* b, int b_is_f16, uint32_t rank, uint32_t d_out, const float* t,
                         float scale, uint32_t rows, float* y, uint32_t y_stride, hipStream_t stream);

// Y[M,N] = X[M,K] . W^T (+ LoRA); X f32 or f16, Y f32.
// gemm_scratch_floats = floats of scratch launch_gemm needs for the shape (0 = none).
// `forced`: 0 = choose by shape, 1 = LDS-staged kernel, 2 = weights-in-registers kernel where supported,
// 3 = few-token kernel, 4 = the weights-in-registers tile at two workgroups per CU (a context's setting).
size_t gemm_scratch_floats(uint32_t n, uint32_t k, uint32_t m, int x_is_f16, bool with_lora, int forced);
// true = launch_gemm serves the shape (with a LoRA epilogue) with the few-token kernel below
bool gemm_takes_few_token_kernel(uint32_t n, uint32_t k, uint32_t m, int x_is_f16, int forced);
void launch_gemm(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m,
                 float* y, const LoraEpilogue& lora, float* scratch, int forced, hipStream_t stream);
int gemm_kernel_choice_default();  // from the environment variable LQ4_GEMM_KERNEL

// Large-shape variant: weights dequantised in registers, only activations staged in LDS.
// Tile 128 tokens x 256 weight rows; gemm_wreg_tiles = workgroups it would launch;
// gemm_wreg_supports = the kernel can run the shape at all.
uint32_t gemm_wreg_tiles(uint32_t n, uint32_t m);
bool gemm_wreg_supports(uint32_t n, uint32_t k, uint32_t m, int x_is_f16);
// A last, partly filled round of tiles is cut into K slices that meet in `partial`
// (gemm_wreg_scratch_floats floats; null = no slicing) and are summed by a second kernel.
size_t gemm_wreg_scratch_floats(uint32_t n, uint32_t k, uint32_t m);
// The same tile at two workgroups per CU, Q4 only: activations packed into scratch first (f16, tile order),
// then the tail's partial tiles behind them; gemm_w2_scratch_bytes covers both.
size_t gemm_w2_scratch_bytes(uint32_t n, uint32_t k, uint32_t m);
bool gemm_w2_wants(uint32_t n, uint32_t k, uint32_t m);
void launch_gemm_w2(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    uint8_t* scratch, hipStream_t stream);
void launch_gemm_wreg(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m,
                      float* y, const LoraEpilogue& lora, float* partial, hipStream_t stream, int fmt = 0);

// Q8_0 sibling format (34-byte blocks: f16 scale + 32 x i8, w = q * d): batch-1 GEMV with x staged
// in LDS (gemv_q8_lds_bytes(k) bytes), and the LDS-staged tile GEMM for everything else.
size_t gemv_q8_lds_bytes(uint32_t k);
void launch_gemv_q8_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream);
void launch_gemm_q8(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    float* scratch, int forced, hipStream_t stream);
// Floats of scratch the sibling tile GEMMs use to cut K on shapes with few tiles (0 = none; a null
// scratch pointer keeps K whole).
size_t gemm_sibling_scratch_floats(int fmt, uint32_t n, uint32_t k, uint32_t m, int forced);  // fmt: 1 = Q8_0, 2 = Q3

// Q3 sibling format (16-byte blocks: f16 scale, f16 bias, 2-bit and 1-bit planes): same pair of paths.
size_t gemv_q3_lds_bytes(uint32_t k);
void launch_gemv_q3_b1(const uint8_t* w, uint32_t n, uint32_t k, const float* x, float* y, hipStream_t stream);
void launch_gemm_q3(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                    float* scratch, int forced, hipStream_t stream);

// Few-token variant (up to 128 tokens): activations packed once into matrix-core operand order
// (gemm_skinny_scratch_bytes bytes at `packed_x`), then a kernel without LDS staging.
bool gemm_skinny_wants(uint32_t n, uint32_t k, uint32_t m);
size_t gemm_skinny_scratch_bytes(uint32_t k, uint32_t m);
// For Q4 and a LoRA rank this accepts, the kernel computes t = A . X itself when LoraEpilogue::a points to A as
// packed (on the host, once) by gemm_skinny_pack_lora_a; t is then not read and no launch for it has to precede.
bool gemm_skinny_computes_t(uint32_t rank, uint32_t m, uint32_t n);
bool gemm_skinny_packs_lora_a(uint32_t rank);  // an adapter of this rank gets a packed copy of A at upload
size_t gemm_skinny_packed_lora_a_bytes(uint32_t k);
void gemm_skinny_pack_lora_a(const void* a_host, int a_is_f16, uint32_t rank, uint32_t k, void* out_host);
// fmt: 0 = Q4 blocks, 1 = Q8_0, 2 = Q3.
// pack = false: `packed_x` already holds the packed image of this x (an earlier call with the same x, K, m and format).
void launch_gemm_skinny(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m, float* y,
                        const LoraEpilogue& lora, void* packed_x, hipStream_t stream, int fmt = 0, bool pack = true);

bool launch_probe_read(const void* p, size_t nbytes, uint32_t grid, uint32_t in_flight, bool strided, bool nontemporal,
                       uint32_t* sink, hipStream_t stream);
void launch_probe_copy(const void* src, void* dst, size_t nbytes, hipStream_t stream);
void launch_dequant(const uint8_t* w, uint32_t n, uint32_t k, float* out, hipStream_t stream);

// With `shared_gate` the table has top_k + 1 slots per token and slot top_k carries expert id `num_experts`
// with weight sigmoid(x[t] . shared_gate) (x: [tokens, hidden]).
void launch_moe_route(const float* logits, uint32_t tokens, uint32_t num_experts, uint32_t top_k,
                      int32_t* ids, float* weights, hipStream_t stream, const float* x = nullptr,
                      const float* shared_gate = nullptr, uint32_t hidden = 0);

// Scratch layout for the grouped MoE path, all sized by the caller:
//   counts  i32 [E]        pairs routed to each expert
//   offsets i32 [E + 1]    exclusive prefix of counts
//   order   i32 [P]        pair indices (token*top_k + slot) sorted by expert, stable
//   h       f32 [P, inter] silu(gate)*up per pair
//   o       f32 [P, hidden] down-projection per pair
struct MoeScratch {
    int32_t* counts;
    int32_t* offsets;
    int32_t* order;
    float* h;
    float* o;
};
void launch_moe_grouped(const uint8_t* gate_up, const uint8_t* down, uint32_t num_experts,
                        uint32_t inter, uint32_t hidden, const float* x, uint32_t tokens,
                        const int32_t* ids, const float* weights, uint32_t top_k, float* y,
                        const MoeScratch& s, hipStream_t stream, const uint8_t* shared_gate_up = nullptr,
                        const uint8_t* shared_down = nullptr);
// With shared tensors (an expert as wide as the routed ones; needs moe_i8_serves(hidden) and
// moe_i8_serves(inter)) ids / weights are [tokens, top_k + 1] as launch_moe_route writes them with a shared
// gate, and the scratch is sized for tokens * (top_k + 1) pairs and num_experts + 1 experts.

// Matrix-core form of the two expert passes (lq4_moe_i8.hip; the activations of a pass are staged in LDS, which
// bounds the reduction length it takes).
bool moe_i8_serves(uint32_t k);
// `ids` not null (up to kMoeIdsMaxPairs pairs and kMoeIdsMaxExperts experts): the kernels find every expert's pairs in
// the routing table themselves (offsets and order are then unused); null: they read the grouping tables.
constexpr uint32_t kMoeIdsMaxPairs = 512, kMoeIdsMaxExperts = 512;
void launch_moe_gate_up_i8(const uint8_t* gate_up, uint32_t num_experts, uint32_t inter, uint32_t hidden, const float* x,
                           uint32_t tokens, uint32_t top_k, const int32_t* offsets, const int32_t* order,
                           const int32_t* ids, float* h, hipStream_t stream, const uint8_t* last_expert = nullptr);
void launch_moe_down_i8(const uint8_t* down, uint32_t num_experts, uint32_t inter, uint32_t hidden, const float* h,
                        uint32_t tokens, uint32_t top_k, const int32_t* offsets, const int32_t* order,
                        const int32_t* ids, float* o, hipStream_t stream, const uint8_t* last_expert = nullptr);
// (`last_expert`: the tensor of expert num_experts - 1 when it does not follow the others in `gate_up` / `down`)

// Exact top-k over n logits (k <= 256): out_logits / out_ids receive the k best in rank order.
// `scratch` must hold topk_scratch_bytes(n, k) bytes; `ticket` is one device word that is zero
// between launches (the kernel counts finished workgroups in it and puts it back to zero).
size_t topk_scratch_bytes(uint32_t n, uint32_t k);
void launch_topk(const float* logits, uint32_t n, uint32_t k, void* scratch, uint32_t* ticket, float* out_logits,
                 uint32_t* out_ids, hipStream_t stream);

// ---- device helpers ---------------------------------------------------------------
// v summed over the four 16-lane rows of a wave: every lane ends with the total of the four lanes
// at its position in a row, (r0 + r1) + (r2 + r3) seen from rows 0/1 and mirrored from rows 2/3, the
// same sums as adding the lanes at xor 16 and then xor 32.  The two row-swap instructions of this
// chip exchange registers directly, where a general lane shuffle goes through the LDS crossbar at
// ~100 cycles of latency each.
__device__ __forceinline__ float sum_over_rows(float v) {
    float a = v, b = v;
    asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));  // a: rows 0 0 2 2, b: rows 1 1 3 3
    v = a + b;
    a = v;
    b = v;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));  // a: low half twice, b: high half twice
    return a + b;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
    // v_cvt_f32_f16 widens exactly, subnormals included (f16 denormals are not flushed
    // in the default HIP float mode).
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16)));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Partial dot product of row `j` of A (f16 or f32, `k` long, k a multiple of 32) with x, for thread
// `t` of `nt`: eight elements per step through 16-byte loads.
__device__ __forceinline__ float lora_a_row_partial(const void* a, int a_is_f16, uint32_t j, uint32_t k,
                                                    const float* __restrict__ x, uint32_t t, uint32_t nt) {
    float p = 0.0f;
    for (uint32_t kk = t * 8; kk < k; kk += nt * 8) {
        const float4 x0 = *reinterpret_cast<const float4*>(x + kk), x1 = *reinterpret_cast<const float4*>(x + kk + 4);
        float av[8];
        if (a_is_f16) {
            struct alignas(16) H8 { _Float16 v[8]; };
            const H8 h = *reinterpret_cast<const H8*>(static_cast<const _Float16*>(a) + static_cast<size_t>(j) * k + kk);
#pragma unroll
            for (int i = 0; i < 8; ++i) av[i] = static_cast<float>(h.v[i]);
        } else {
            const float4* ap = reinterpret_cast<const float4*>(static_cast<const float*>(a) + static_cast<size_t>(j) * k + kk);
            const float4 a0 = ap[0], a1 = ap[1];
            av[0] = a0.x; av[1] = a0.y; av[2] = a0.z; av[3] = a0.w;
            av[4] = a1.x; av[5] = a1.y; av[6] = a1.z; av[7] = a1.w;
        }
        p = fmaf(av[0], x0.x, p); p = fmaf(av[1], x0.y, p); p = fmaf(av[2], x0.z, p); p = fmaf(av[3], x0.w, p);
        p = fmaf(av[4], x1.x, p); p = fmaf(av[5], x1.y, p); p = fmaf(av[6], x1.z, p); p = fmaf(av[7], x1.w, p);
    }
    return p;
}

// The tag of a launch: where its dispatch packet lies in the queue's ring (a 64-byte slot of it; the address is an
// input register of every wave).  Every workgroup of one launch sees the same packet, the next launch on the queue
// the next slot, also when a captured graph is replayed (the packets are written again); other queues of the
// process have their rings elsewhere.  31 bits of the slot number, the top bit set so that a zeroed word never
// matches.  A launch could only take another launch's words for its own if that one lay a whole number of laps of
// the ring earlier AND no launch in between had published to the same slots.
__device__ __forceinline__ uint32_t launch_tag() {
    const uintptr_t packet = reinterpret_cast<uintptr_t>(__builtin_amdgcn_dispatch_ptr());
    return static_cast<uint32_t>(packet >> 6) | 0x80000000u;
}

// Shared inner loop of the GEMV-class kernels.  One wave accumulates R weight rows
// (rowp[r] = first block of row r) against NB activation rows (xrow[b]), each of
// `nb` blocks / nb*32 floats.  Lane l handles packed dword (l & 3) of blocks
// (l >> 2), (l >> 2) + 16, ...: 8 consecutive weights against 8 consecutive
// activations.  acc holds per-lane partial sums; the caller reduces across the wave.
// Every xrow[b] must be 16-byte aligned.
template <int R, int NB>
__device__ __forceinline__ void q4_rows_dot(const uint8_t* const (&rowp)[R], uint32_t nb,
                                            const float* const (&xrow)[NB], int lane,
                                            float (&acc)[R][NB]) {
    const int il = lane & 3;
    for (uint32_t ib = lane >> 2; ib < nb; ib += 16) {
        float xv[NB][8];
        float xs[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const float4* xp = reinterpret_cast<const float4*>(xrow[b] + ib * kBlockWeights + il * 8);
            const float4 lo = xp[0], hi = xp[1];
            xv[b][0] = lo.x; xv[b][1] = lo.y; xv[b][2] = lo.z; xv[b][3] = lo.w;
            xv[b][4] = hi.x; xv[b][5] = hi.y; xv[b][6] = hi.z; xv[b][7] = hi.w;
            xs[b] = ((lo.x + lo.y) + (lo.z + lo.w)) + ((hi.x + hi.y) + (hi.z + hi.w));
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t* blk =
                reinterpret_cast<const uint32_t*>(rowp[r] + static_cast<size_t>(ib) * kBlockBytes);
            const uint32_t sb = blk[0];
            const uint32_t q = blk[1 + il];
            const float d = f16_bits_to_f32(sb & 0xffffu);
            const float bias = f16_bits_to_f32(sb >> 16);
            float qf[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) qf[i] = static_cast<float>((q >> (4 * i)) & 0xfu);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float s = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) s = fmaf(qf[i], xv[b][i], s);
                acc[r][b] = fmaf(s, d, fmaf(bias, xs[b], acc[r][b]));
            }
        }
    }
}

}  // namespace lq4
