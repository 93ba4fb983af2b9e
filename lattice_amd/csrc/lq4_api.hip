// C ABI of liblattice_hip_q4.so (declared in include/lattice_hip_q4.h): argument and
// bounds checking, device residency of weights and LoRA factors, and kernel dispatch.
// Nothing here falls back to the CPU: without a working HIP device every entry point
// that would launch returns LQ4_E_HIP.
#include "../../include/lattice_hip_q4.h"

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "lq4_internal.hpp"

using namespace lq4;

struct lq4_ctx {
    int device;
    float* lora_t;        // [kLoraTRows, kMaxLoraRank] f32: A.x of the call in flight
    uint8_t* static_scratch;  // this device's copy of `scratch` below (lq4_lm_head_topk_static)
    uint8_t* moe_scratch; // grown on demand
    uint32_t* topk_ticket; // finished-workgroup count of the top-k kernel, zero between launches
    uint32_t* lora_sync;   // fall-back count (word 2) and, from word 64 on, the slots of the batch-1 GEMV that computes A.x itself (same allocation)
    unsigned long long* lora_slots_rows;  // [kMaxLoraRank][8]: the slots of the 2..8-row GEMV that computes A.x itself (same allocation)
    bool lora_in_kernel;
    uint32_t lora_spin_limit;  // polls a weight wave spends on those counters before it computes A.x alone
    size_t moe_scratch_bytes;
    uint8_t* shared_scratch;  // intermediates of calls that run lq4_gemv / lq4_gemm in between (those use moe_scratch)
    size_t shared_scratch_bytes;
    // Buffers the growable scratch outgrew: launches already queued (or captured into a graph) may
    // still use them, so they are only released with the context.
    std::vector<void*> retired;
    // lq4_gemv_chain: the result vectors of steps whose result nobody asked for
    uint8_t* chain_scratch;
    size_t chain_scratch_bytes;
    uint32_t cu_count;
    // The stream of the last call that used the context's shared state (scratch buffers, hand-over words):
    // a call on another stream makes its stream wait for everything queued on that one so far, so that calls
    // alternating between streams are ordered instead of racing on that state.
    hipStream_t state_stream;
    bool state_stream_known;
    hipEvent_t state_event;  // recorded on the previous stream when a call arrives on another one
    int gemm_kernel;         // lq4_set_gemm_kernel
    int gemv_kernel;         // lq4_set_gemv_kernel: which kernel serves a plain one-token GEMV
    int gemv_i8;             // LQ4_GEMV_I8: 1 = 3..8 rows of small matrices take the integer matrix-core kernel (default),
                             // 0 = never, 2 = 2..8 rows of every matrix it can serve (tests)
    lq4_path_counters counters;
};

struct lq4_weight {
    lq4_ctx* ctx;
    uint8_t* base;  // byte 0 of the uploaded buffer
    size_t nbytes;
    uint64_t payload_offset;
    bool owned;
};

struct lq4_lora {
    lq4_ctx* ctx;
    void* a;  // [rank, d_in]
    void* b;  // [d_out, rank]
    int is_f16;
    uint32_t rank, d_in, d_out;
    void* a_packed;  // A as the few-token GEMM's operand (ranks it accepts; else null): that kernel's in-launch A . X
};

namespace {

constexpr size_t kFusedPrologueBytes = 64u << 10;  // lq4_gemv_fused_batch: see there
constexpr uint32_t kSharedB1MaxTokens = 8;  // shared expert alone through the per-pair kernels up to here (route + routed + shared as three calls: 8 tokens 56.0 -> 51.7 us, 16 tokens 68.5 -> 66.6, 32 tokens 89.3 -> 94.3)
constexpr uint32_t kMoeB1MaxTokens = 8;  // per-pair expert kernels up to here (measured: 1 / 2 / 4 / 8 / 16 tokens 27.5 / 30.5 / 43.2 / 45.1 / 48.6 us grouped, 13.7 / 18.3 / 25.9 / 39.1 / 65.0 per pair)
constexpr uint32_t kMoeSharedGroupedMaxTokens = 384;  // lq4_moe_ffn: shared expert as one more expert of the grouped kernels up to here (level at 512)
constexpr uint32_t kMultiMaxRows = 128;  // lq4_gemv_multi: up to the few-token GEMM's range
constexpr uint32_t kLoraTRows = 4096;  // most rows one LoRA-fused call may carry

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return code;
}

#define LQ4_HIP(call)                                                                     \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) return fail(LQ4_E_HIP, "%s: %s", #call, hipGetErrorString(e_)); \
    } while (0)

struct DeviceGuard {
    int prev = -1;
    bool ok = true;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        if (prev != dev) ok = hipSetDevice(dev) == hipSuccess;
        // An error some earlier, unrelated runtime call left behind in this thread must not be
        // reported by the launch check of this entry point.
        if (ok) (void)hipGetLastError();
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

float half_bits_to_float(uint16_t h) {
    // exact widening incl. subnormals (crates/inference/src/weights/half_bits.rs:24-53)
    const uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1fu, frac = h & 0x3ffu;
    float mag;
    if (exp == 0) mag = std::ldexp(static_cast<float>(frac), -24);
    else if (exp == 0x1f) mag = frac ? NAN : INFINITY;
    else mag = std::ldexp(static_cast<float>(frac | 0x400u), static_cast<int>(exp) - 25);
    return sign ? -mag : mag;
}

// Checks K and that W[n,k] lies inside the buffer; yields the device address of W.
int resolve_weight(const lq4_weight* w, uint64_t extra, uint32_t n, uint32_t k,
                   const uint8_t** out) {
    if (!w) return fail(LQ4_E_INVALID, "weight handle is null");
    if (k == 0 || k % kBlockWeights != 0)
        return fail(LQ4_E_INVALID, "Q4 matmul requires K to be non-zero and divisible by 32, got %u", k);
    const uint64_t need = static_cast<uint64_t>(n) * (k / kBlockWeights) * kBlockBytes;
    const uint64_t start = w->payload_offset + extra;
    if (start > w->nbytes || need > w->nbytes - start)
        return fail(LQ4_E_INVALID, "W[%u,%u] at byte %llu needs %llu bytes but the buffer holds %zu", n, k,
                    static_cast<unsigned long long>(start), static_cast<unsigned long long>(need), w->nbytes);
    if (start % 4 != 0) return fail(LQ4_E_INVALID, "weight byte offset %llu is not 4-byte aligned",
                                    static_cast<unsigned long long>(start));
    *out = w->base + start;
    return LQ4_OK;
}

// The same for a buffer of sibling-format blocks: Q8_0 (34 bytes, 2-byte aligned) or Q3 (16 bytes,
// 4-byte aligned).
int resolve_weight_sibling(const lq4_weight* w, uint64_t extra, uint32_t n, uint32_t k, const char* fmt,
                           uint32_t block_bytes, uint32_t align, const uint8_t** out) {
    if (!w) return fail(LQ4_E_INVALID, "weight handle is null");
    if (k == 0 || k % kBlockWeights != 0)
        return fail(LQ4_E_INVALID, "%s matmul requires K to be non-zero and divisible by 32, got %u", fmt, k);
    const uint64_t need = static_cast<uint64_t>(n) * (k / kBlockWeights) * block_bytes;
    const uint64_t start = w->payload_offset + extra;
    if (start > w->nbytes || need > w->nbytes - start)
        return fail(LQ4_E_INVALID, "%s W[%u,%u] at byte %llu needs %llu bytes but the buffer holds %zu", fmt, n, k,
                    static_cast<unsigned long long>(start), static_cast<unsigned long long>(need), w->nbytes);
    if (start % align != 0) return fail(LQ4_E_INVALID, "%s weight byte offset %llu is not %u-byte aligned", fmt,
                                        static_cast<unsigned long long>(start), align);
    *out = w->base + start;
    return LQ4_OK;
}

int resolve_weight_q8(const lq4_weight* w, uint64_t extra, uint32_t n, uint32_t k, const uint8_t** out) {
    return resolve_weight_sibling(w, extra, n, k, "Q8", 34, 2, out);
}

int resolve_lora(const lq4_ctx* ctx, const lq4_lora* l, float scale, uint32_t n, uint32_t k,
                 uint32_t rows, LoraEpilogue* out) {
    *out = LoraEpilogue{nullptr, nullptr, 0, 0, 0.0f};
    if (!l) return LQ4_OK;
    if (l->d_in != k || l->d_out != n)
        return fail(LQ4_E_INVALID, "LoRA is [%u -> %u] but the projection is [%u -> %u]", l->d_in, l->d_out, k, n);
    if (rows > kLoraTRows) return fail(LQ4_E_UNSUPPORTED, "LoRA-fused call limited to %u rows, got %u", kLoraTRows, rows);
    out->b = l->b;
    out->t = ctx->lora_t;
    out->rank = l->rank;
    out->b_is_f16 = l->is_f16;
    out->scale = scale;
    return LQ4_OK;
}

}  // namespace

extern "C" {

const char* lq4_last_error(void) { return g_err; }
const char* lq4_version(void) { return "lattice-hip-q4 0.1 (gfx950)"; }

// Scratch of lq4_lm_head_topk_static, in the code object's own data so that entry point never
// allocates: the logits of one lm_head pass, then the top-k candidate buffers.  Every GPU the
// library runs on holds one copy until the process ends; host code reaches it only through the
// address hipGetSymbolAddress returns for the current device (kept in the context).
constexpr size_t kStaticScratchBytes = LQ4_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

int lq4_ctx_create(int device_ordinal, lq4_ctx** out) {
    if (!out) return fail(LQ4_E_INVALID, "out is null");
    *out = nullptr;
    int count = 0;
    LQ4_HIP(hipGetDeviceCount(&count));
    if (device_ordinal < 0 || device_ordinal >= count)
        return fail(LQ4_E_INVALID, "device %d out of range (%d visible)", device_ordinal, count);
    DeviceGuard g(device_ordinal);
    if (!g.ok) return fail(LQ4_E_HIP, "hipSetDevice(%d) failed", device_ordinal);
    lq4_ctx* c = new (std::nothrow) lq4_ctx();
    if (!c) return fail(LQ4_E_NOMEM, "out of host memory");
    c->device = device_ordinal;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&c->lora_t), sizeof(float) * kLoraTRows * kMaxLoraRank);
    if (e != hipSuccess) {
        delete c;
        return fail(LQ4_E_HIP, "hipMalloc(lora scratch): %s", hipGetErrorString(e));
    }
    // 256 B of top-k ticket, 256 B for the LoRA fall-back count, 512 B of LoRA slots for one activation row, 4 KB
    // of them for up to eight rows (a zeroed slot matches no launch: every tag has its top bit set)
    e = hipMalloc(reinterpret_cast<void**>(&c->topk_ticket), 1024 + 8 * kMaxLoraRank * 8);
    if (e == hipSuccess) e = hipMemset(c->topk_ticket, 0, 1024 + 8 * kMaxLoraRank * 8);
    if (e != hipSuccess) {
        (void)hipFree(c->topk_ticket);
        (void)hipFree(c->lora_t);
        delete c;
        return fail(LQ4_E_HIP, "hipMalloc(top-k ticket): %s", hipGetErrorString(e));
    }
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&c->static_scratch), HIP_SYMBOL(scratch));
    if (e != hipSuccess || !c->static_scratch) {
        (void)hipFree(c->topk_ticket);
        (void)hipFree(c->lora_t);
        delete c;
        return fail(LQ4_E_HIP, "hipGetSymbolAddress(static scratch): %s", hipGetErrorString(e));
    }
    c->lora_sync = c->topk_ticket + 64;
    c->lora_slots_rows = reinterpret_cast<unsigned long long*>(c->topk_ticket + 256);
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device_ordinal);
    if (e != hipSuccess) {
        (void)hipFree(c->topk_ticket);
        (void)hipFree(c->lora_t);
        delete c;
        return fail(LQ4_E_HIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    }
    c->cu_count = static_cast<uint32_t>(prop.multiProcessorCount);
    e = hipEventCreateWithFlags(&c->state_event, hipEventDisableTiming);
    if (e != hipSuccess) {
        (void)hipFree(c->topk_ticket);
        (void)hipFree(c->lora_t);
        delete c;
        return fail(LQ4_E_HIP, "hipEventCreate: %s", hipGetErrorString(e));
    }
    c->gemm_kernel = gemm_kernel_choice_default();
    c->gemv_kernel = getenv("LQ4_GEMV_KERNEL") ? atoi(getenv("LQ4_GEMV_KERNEL")) : 0;
    if (c->gemv_kernel < 0 || c->gemv_kernel > 2) c->gemv_kernel = 0;
    c->gemv_i8 = getenv("LQ4_GEMV_I8") ? atoi(getenv("LQ4_GEMV_I8")) : 1;
    if (c->gemv_i8 < 0 || c->gemv_i8 > 2) c->gemv_i8 = 1;
    // LQ4_LORA_SPIN_LIMIT: 0 makes every weight wave compute A.x itself (the path a wave takes when
    // the producers are late), "off" restores the separate A.x launch
    c->lora_spin_limit = 512;
    c->lora_in_kernel = true;
    if (const char* env = getenv("LQ4_LORA_SPIN_LIMIT")) {
        if (!strcmp(env, "off")) c->lora_in_kernel = false;
        else c->lora_spin_limit = static_cast<uint32_t>(strtoul(env, nullptr, 10));
    }
    *out = c;
    return LQ4_OK;
}

int lq4_ctx_destroy(lq4_ctx* ctx) {
    if (!ctx) return LQ4_OK;
    DeviceGuard g(ctx->device);
    (void)hipFree(ctx->lora_t);
    (void)hipFree(ctx->topk_ticket);
    if (ctx->moe_scratch) (void)hipFree(ctx->moe_scratch);
    if (ctx->shared_scratch) (void)hipFree(ctx->shared_scratch);
    if (ctx->chain_scratch) (void)hipFree(ctx->chain_scratch);
    for (void* p : ctx->retired) (void)hipFree(p);
    (void)hipEventDestroy(ctx->state_event);
    delete ctx;
    return LQ4_OK;
}

int lq4_sync(lq4_ctx* ctx, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    LQ4_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return LQ4_OK;
}

int lq4_validate_blocks(const uint8_t* p, size_t nbytes, int64_t* bad_block, int* reason) {
    if (!p && nbytes) return fail(LQ4_E_INVALID, "payload is null");
    const size_t nb = nbytes / kBlockBytes;
    for (size_t i = 0; i < nb; ++i) {
        const uint8_t* c = p + i * kBlockBytes;
        const float scale = half_bits_to_float(static_cast<uint16_t>(c[0] | (c[1] << 8)));
        const float bias = half_bits_to_float(static_cast<uint16_t>(c[2] | (c[3] << 8)));
        int why = 0;
        if (!std::isfinite(scale) || scale <= 0.0f) why = 1;
        else if (!std::isfinite(bias)) why = 2;
        if (why) {
            if (bad_block) *bad_block = static_cast<int64_t>(i);
            if (reason) *reason = why;
            return why == 1
                       ? fail(LQ4_E_BLOCK, "Q4 block %zu has invalid scale %g; scale must be finite and strictly positive", i, scale)
                       : fail(LQ4_E_BLOCK, "Q4 block %zu has non-finite bias %g", i, bias);
        }
    }
    if (bad_block) *bad_block = -1;
    if (reason) *reason = 0;
    return LQ4_OK;
}

int lq4_weight_upload(lq4_ctx* ctx, const uint8_t* host_bytes, size_t nbytes, uint64_t payload_offset,
                      int validate, lq4_weight** out) {
    if (!ctx || !host_bytes || !out) return fail(LQ4_E_INVALID, "null argument");
    *out = nullptr;
    if (payload_offset > nbytes) return fail(LQ4_E_INVALID, "payload_offset %llu beyond buffer length %zu",
                                             static_cast<unsigned long long>(payload_offset), nbytes);
    if (payload_offset % 4) return fail(LQ4_E_INVALID, "payload_offset must be 4-byte aligned");
    if (validate) {
        int rc = lq4_validate_blocks(host_bytes + payload_offset, nbytes - payload_offset, nullptr, nullptr);
        if (rc) return rc;
    }
    DeviceGuard g(ctx->device);
    lq4_weight* w = new (std::nothrow) lq4_weight{ctx, nullptr, nbytes, payload_offset, true};
    if (!w) return fail(LQ4_E_NOMEM, "out of host memory");
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&w->base), nbytes ? nbytes : 4);
    if (e == hipSuccess && nbytes) e = hipMemcpy(w->base, host_bytes, nbytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        if (w->base) (void)hipFree(w->base);
        delete w;
        return fail(LQ4_E_HIP, "weight upload (%zu bytes): %s", nbytes, hipGetErrorString(e));
    }
    *out = w;
    return LQ4_OK;
}

int lq4_weight_wrap(lq4_ctx* ctx, const void* blocks_dev, size_t nbytes, uint64_t payload_offset,
                    lq4_weight** out) {
    if (!ctx || !blocks_dev || !out) return fail(LQ4_E_INVALID, "null argument");
    if (payload_offset > nbytes || payload_offset % 4) return fail(LQ4_E_INVALID, "bad payload_offset");
    if (reinterpret_cast<uintptr_t>(blocks_dev) % 4) return fail(LQ4_E_INVALID, "device buffer must be 4-byte aligned");
    lq4_weight* w = new (std::nothrow) lq4_weight{
        ctx, const_cast<uint8_t*>(static_cast<const uint8_t*>(blocks_dev)), nbytes, payload_offset, false};
    if (!w) return fail(LQ4_E_NOMEM, "out of host memory");
    *out = w;
    return LQ4_OK;
}

int lq4_weight_free(lq4_weight* w) {
    if (!w) return LQ4_OK;
    if (w->owned) {
        DeviceGuard g(w->ctx->device);
        (void)hipFree(w->base);
    }
    delete w;
    return LQ4_OK;
}

int lq4_weight_info(const lq4_weight* w, const void** base_dev, size_t* nbytes, uint64_t* payload_offset) {
    if (!w) return fail(LQ4_E_INVALID, "weight handle is null");
    if (base_dev) *base_dev = w->base;
    if (nbytes) *nbytes = w->nbytes;
    if (payload_offset) *payload_offset = w->payload_offset;
    return LQ4_OK;
}

int lq4_lora_upload(lq4_ctx* ctx, const void* a_host, const void* b_host, int dtype, uint32_t rank,
                    uint32_t d_in, uint32_t d_out, lq4_lora** out) {
    if (!ctx || !a_host || !b_host || !out) return fail(LQ4_E_INVALID, "null argument");
    *out = nullptr;
    if (dtype != LQ4_F32 && dtype != LQ4_F16) return fail(LQ4_E_INVALID, "dtype must be LQ4_F32 or LQ4_F16");
    if (rank == 0 || d_in == 0 || d_out == 0) return fail(LQ4_E_INVALID, "LoRA rank/d_in/d_out must be non-zero");
    if (rank > kMaxLoraRank) return fail(LQ4_E_UNSUPPORTED, "LoRA rank %u above the supported maximum %d", rank, kMaxLoraRank);
    const size_t es = dtype == LQ4_F16 ? 2 : 4;
    DeviceGuard g(ctx->device);
    lq4_lora* l = new (std::nothrow) lq4_lora{ctx, nullptr, nullptr, dtype == LQ4_F16, rank, d_in, d_out, nullptr};
    if (!l) return fail(LQ4_E_NOMEM, "out of host memory");
    const size_t a_bytes = es * rank * d_in, b_bytes = es * d_out * rank;
    hipError_t e = hipMalloc(&l->a, a_bytes);
    if (e == hipSuccess) e = hipMalloc(&l->b, b_bytes);
    if (e == hipSuccess) e = hipMemcpy(l->a, a_host, a_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(l->b, b_host, b_bytes, hipMemcpyHostToDevice);
    if (e == hipSuccess && gemm_skinny_packs_lora_a(rank)) {  // A once more, as the few-token GEMM's own operand
        const size_t bytes = gemm_skinny_packed_lora_a_bytes(d_in);
        void* host = malloc(bytes);
        if (!host) {
            (void)hipFree(l->a);
            (void)hipFree(l->b);
            delete l;
            return fail(LQ4_E_NOMEM, "out of host memory");
        }
        gemm_skinny_pack_lora_a(a_host, dtype == LQ4_F16, rank, d_in, host);
        e = hipMalloc(&l->a_packed, bytes);
        if (e == hipSuccess) e = hipMemcpy(l->a_packed, host, bytes, hipMemcpyHostToDevice);
        free(host);
    }
    if (e != hipSuccess) {
        if (l->a_packed) (void)hipFree(l->a_packed);
        if (l->a) (void)hipFree(l->a);
        if (l->b) (void)hipFree(l->b);
        delete l;
        return fail(LQ4_E_HIP, "LoRA upload: %s", hipGetErrorString(e));
    }
    *out = l;
    return LQ4_OK;
}

int lq4_lora_free(lq4_lora* l) {
    if (!l) return LQ4_OK;
    DeviceGuard g(l->ctx->device);
    (void)hipFree(l->a_packed);
    (void)hipFree(l->a);
    (void)hipFree(l->b);
    delete l;
    return LQ4_OK;
}

static int ensure_scratch(lq4_ctx* ctx, size_t bytes, hipStream_t stream);
static int enter_shared_state(lq4_ctx* ctx, hipStream_t stream);

// y = W . x for one token without LoRA: the LDS-ring kernel where it is the faster one (or where the context asks
// for it and the shape fits), else the lane-owns-block kernel.  Both give the same contract.
static void plain_gemv_one_token(lq4_ctx* ctx, const uint8_t* wp, uint32_t n, uint32_t k, const float* x, float* y,
                                 hipStream_t s) {
    const bool ring = ctx->gemv_kernel == LQ4_GEMV_KERNEL_LDS_RING
                          ? gemv_dma_serves(n, k, ctx->cu_count)
                          : ctx->gemv_kernel == LQ4_GEMV_KERNEL_AUTO && gemv_dma_pays(n, k, ctx->cu_count);
    if (ring) {
        launch_gemv_dma(wp, n, k, x, y, ctx->cu_count, s);
    } else {
        const LoraEpilogue none{};
        launch_gemv(wp, n, k, x, k, 1, y, n, none, s);
    }
    ctx->counters.gemv++;
}

// 2..8 rows on the integer matrix-core kernel: three to eight rows of a matrix of up to 4096 x 2048; five to eight
// rows of a tall matrix of short rows (12288 x 2048 9.6-10.0 -> 8.7-8.8 us, 16384 x 2048 11.0-11.6 -> 8.8-9.0,
// 9728 x 2560 12.0-12.6 -> 10.0-10.1; at 2..4 rows the 4x4x4 kernel is ahead there, 6.3-7.3 us against 7.8); or, for
// the tests, whatever it can hold.
static bool gemv_takes_i8(const lq4_ctx* ctx, uint32_t n, uint32_t k, uint32_t batch) {
    const bool small = batch >= 3 && k <= 2048 && n <= 4096;
    const bool tall = batch >= 5 && gemv_i8_many_short_rows(n, k, ctx->cu_count);
    return batch >= 2 && batch <= 8 && ctx->gemv_i8 && (ctx->gemv_i8 == 2 || small || tall) &&
           gemv_i8_serves(n, k, batch, ctx->cu_count);
}

// Above four activation rows the few-token matrix-core kernel (operands packed once, eight K
// slices per workgroup) overtakes the 4x4x4 GEMV kernel: always from nine rows; from five for
// mid-sized matrices only (measured: behind for 512 x 2048, where its two launches dominate,
// and for 12288 x 2048, where the GEMV kernel's grid already fills the chip), and not where the integer
// matrix-core kernel serves (3072 x 2048 at 5..8 rows 5.8-5.9 us here, 5.4-5.5 there; 4096 x 2048 6.2 / 5.5).
static bool gemv_takes_few_token_gemm(const lq4_ctx* ctx, uint32_t n, uint32_t k, uint32_t batch) {
    const uint64_t weights = static_cast<uint64_t>(n) * k;
    // (not for up to 2048 rows while the GEMV kernel can stage the activations: its eight-wave
    // workgroups then win, 2048 x 6144 at 5..8 rows 9.5 -> 7.2..8.2 us)
    const bool narrow = n <= 2048 && gemv_mfma_lds_bytes(k, batch < 8 ? batch : 8) <= 150 * 1024;
    return batch >= 9 || (batch >= 5 && n < 8192 && !narrow && weights >= 6000000 && !gemv_takes_i8(ctx, n, k, batch));
}

// The routing of lq4_gemv once the LoRA factor t (if any) is in ep, or ep.a says that the kernel which serves the
// shape computes it: which kernel serves (batch, n, k).
// `x_packed` (may be null): calls in a row on the same x, K and batch share the few-token GEMM's packed activations;
// true once a call has packed them into the context's scratch.
static int gemv_dispatch(lq4_ctx* ctx, const uint8_t* wp, uint32_t n, uint32_t k, const float* x_dev, uint32_t batch,
                         float* y_dev, const LoraEpilogue& ep, hipStream_t s, bool* x_packed = nullptr) {
    int rc;
    if (gemv_takes_few_token_gemm(ctx, n, k, batch)) {
        rc = ensure_scratch(ctx, gemm_skinny_scratch_bytes(k, batch), s);
        if (rc) return rc;
        launch_gemm_skinny(wp, n, k, x_dev, 0, batch, y_dev, ep, ctx->moe_scratch, s, 0, !(x_packed && *x_packed));
        if (x_packed) *x_packed = true;
        ctx->counters.gemm++;
    } else if (batch == 1 && !ep.rank) {
        plain_gemv_one_token(ctx, wp, n, k, x_dev, y_dev, s);
    } else if (gemv_takes_i8(ctx, n, k, batch)) {
        // Three to eight rows of a matrix of up to 4096 x 2048: the integer matrix-core kernel, which is as fast as
        // or faster than the 4x4x4 kernel there (512 x 2048: 4.33 -> 4.09 us at four rows, 4.71 -> 4.53 at eight;
        // 2048 x 2048: 4.67 -> 4.54, 5.09 -> 4.98; 3072 x 2048 at four rows 5.58 -> 4.82) and keeps 24 (up to four rows)
        // or 16 bits of every activation below its block's maximum instead of rounding it to f16.  Behind on long rows
        // and many rows (2048 x 6144 at eight rows 8.7 -> 10.4 us, 12288 x 2048 at four 7.8 -> 8.8), which stay where
        // they were.  With a LoRA epilogue alike (q+v of the 2B model at eight rows 17.6 -> 16.2 us), so that a
        // projection is served by the same arithmetic with and without its adapter.
        launch_gemv_i8(wp, n, k, x_dev, k, batch, y_dev, n, ep, ctx->cu_count, s);
        ctx->counters.gemv++;
    } else {
        launch_gemv(wp, n, k, x_dev, k, batch, y_dev, n, ep, s);
        ctx->counters.gemv++;
    }
    return LQ4_OK;
}

int lq4_gemv(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
             const float* x_dev, uint32_t batch, float* y_dev, const lq4_lora* lora, float lora_scale,
             void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (batch == 0 || n == 0) return LQ4_OK;
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    if (!x_dev || !y_dev) return fail(LQ4_E_INVALID, "x/y device pointer is null");
    if (batch > kMaxGemvBatch) return fail(LQ4_E_INVALID, "lq4_gemv batch %u above %d; use lq4_gemm", batch, kMaxGemvBatch);
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    LoraEpilogue ep;
    rc = resolve_lora(ctx, lora, lora_scale, n, k, batch, &ep);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (ep.rank) {  // the A.x buffer (and, for one token, the hand-over words) belong to the context
        rc = enter_shared_state(ctx, s);
        if (rc) return rc;
    }
    if (ep.rank && batch == 1 && ctx->lora_in_kernel && gemv_b1_lds_bytes(k) <= 128 * 1024) {
        // one token: the GEMV launch computes A.x in its first `rank` workgroups
        ep.a = lora->a;
        ep.slots = reinterpret_cast<unsigned long long*>(ctx->lora_sync + 64);
        ep.sync = ctx->lora_sync;
        ep.spin_limit = ctx->lora_spin_limit;
    } else if (ep.rank && batch > 1 && gemv_takes_few_token_gemm(ctx, n, k, batch) && gemm_skinny_computes_t(ep.rank, batch, n)) {
        ep.a = lora->a_packed;  // the few-token GEMM computes A.x for its token tile itself
    } else if (ep.rank && ctx->lora_in_kernel && gemv_takes_i8(ctx, n, k, batch) &&
               gemv_i8_lora_in_launch(n, k, batch, ep.rank, ctx->cu_count)) {
        // 2..8 rows: `rank` producer workgroups of the launch, on CUs the matrix leaves idle
        ep.a = lora->a;
        ep.slots = ctx->lora_slots_rows;
        ep.sync = ctx->lora_sync;
        ep.spin_limit = ctx->lora_spin_limit;
    } else if (ep.rank) {
        launch_lora_a(lora->a, lora->is_f16, lora->rank, k, x_dev, 0, k, batch, ctx->lora_t, s);
        ctx->counters.lora_a++;
    }
    rc = gemv_dispatch(ctx, wp, n, k, x_dev, batch, y_dev, ep, s);
    if (rc) return rc;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_gemv_multi(lq4_ctx* ctx, const lq4_projection* proj, uint32_t count, uint32_t k, const float* x_dev,
                   uint32_t batch, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (count == 0 || batch == 0) return LQ4_OK;
    if (!proj) return fail(LQ4_E_INVALID, "proj is null");
    if (count > LQ4_MAX_PROJECTIONS) return fail(LQ4_E_INVALID, "%u projections, at most %d a call", count, LQ4_MAX_PROJECTIONS);
    if (batch > kMultiMaxRows) return fail(LQ4_E_INVALID, "lq4_gemv_multi batch %u above %u; use lq4_gemm", batch, kMultiMaxRows);
    if (!x_dev) return fail(LQ4_E_INVALID, "x device pointer is null");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    // every projection is checked before anything is launched: a call fails whole or not at all
    const uint8_t* wp[LQ4_MAX_PROJECTIONS];
    LoraEpilogue ep[LQ4_MAX_PROJECTIONS];
    MultiViews mv{};
    LoraAViews av{};
    uint32_t with_lora = 0, total_rank = 0;
    for (uint32_t i = 0; i < count; ++i) {
        const lq4_projection& p = proj[i];
        if (p.n == 0) continue;
        int rc = resolve_weight(p.w, p.w_extra_offset, p.n, k, &wp[i]);
        if (rc) return rc;
        if (!p.y_dev) return fail(LQ4_E_INVALID, "projection %u: y device pointer is null", i);
        if (reinterpret_cast<uintptr_t>(p.y_dev) % 4) return fail(LQ4_E_INVALID, "projection %u: y must be 4-byte aligned", i);
        rc = resolve_lora(ctx, p.lora, p.lora_scale, p.n, k, batch, &ep[i]);
        if (rc) return rc;
        const uint32_t v = mv.count++;
        if (static_cast<uint64_t>(mv.begin[v]) + p.n > 0xFFFFFFFFull) return fail(LQ4_E_INVALID, "more than 2^32 - 1 rows in all");
        mv.begin[v + 1] = mv.begin[v] + p.n;
        mv.w[v] = wp[i];
        mv.y[v] = p.y_dev;
        // view v keeps its A . x in its own part of the context's buffer: [batch, rank] from row v * batch on
        float* t = ctx->lora_t + static_cast<size_t>(v) * batch * kMaxLoraRank;
        ep[i].t = t;
        mv.b[v] = ep[i].b;
        mv.t[v] = t;
        mv.rank[v] = ep[i].rank;
        mv.b_is_f16[v] = ep[i].b_is_f16;
        mv.scale[v] = ep[i].scale;
        av.a[v] = ep[i].rank ? p.lora->a : nullptr;
        av.t[v] = t;
        av.rank[v] = ep[i].rank;
        av.a_is_f16[v] = ep[i].b_is_f16;
        mv.a[v] = av.a[v];
        mv.t_off[v] = total_rank;
        total_rank += ep[i].rank;
        with_lora += ep[i].rank != 0;
    }
    av.count = mv.count;
    if (mv.count == 0) return LQ4_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (batch > kMaxGemvBatch) {
        // 17..128 rows: lq4_gemm's routing projection by projection.  Those the few-token GEMM serves share one packed
        // image of x (packed by the first of them) and compute their A . X themselves where that kernel can.
        if (with_lora) {
            const int rc = enter_shared_state(ctx, s);
            if (rc) return rc;
        }
        bool x_packed = false;
        for (uint32_t i = 0; i < count; ++i) {
            const lq4_projection& p = proj[i];
            if (p.n == 0) continue;
            const bool few = gemm_takes_few_token_kernel(p.n, k, batch, 0, ctx->gemm_kernel);
            LoraEpilogue e = ep[i];
            if (e.rank && few && gemm_skinny_computes_t(e.rank, batch, p.n)) {
                e.a = p.lora->a_packed;
            } else if (e.rank) {
                e.t = ctx->lora_t;  // one after the other on this stream
                launch_lora_a(p.lora->a, p.lora->is_f16, e.rank, k, x_dev, 0, k, batch, ctx->lora_t, s);
                ctx->counters.lora_a++;
            }
            const size_t scratch_bytes = gemm_scratch_floats(p.n, k, batch, 0, e.rank != 0, ctx->gemm_kernel) * sizeof(float);
            if (scratch_bytes) {
                const int rc = ensure_scratch(ctx, scratch_bytes, s);
                if (rc) return rc;
            }
            if (few) {
                launch_gemm_skinny(wp[i], p.n, k, x_dev, 0, batch, p.y_dev, e, ctx->moe_scratch, s, 0, !x_packed);
                x_packed = true;
            } else {
                launch_gemm(wp[i], p.n, k, x_dev, 0, batch, p.y_dev, e,
                            scratch_bytes ? reinterpret_cast<float*>(ctx->moe_scratch) : nullptr, ctx->gemm_kernel, s);
                x_packed = false;  // (that kernel's partial tiles share the scratch)
            }
            ctx->counters.gemm++;
        }
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    const bool stacked = batch == 1 && (mv.count > 1 || with_lora) && gemv_multi_serves(mv, k);
    // one token: the stacked launch computes every A_v . x in producer workgroups of its own (lane l of a weight
    // wave holds the factor of stacked row l, hence at most 64 rows of A in all)
    const bool in_launch = stacked && with_lora && ctx->lora_in_kernel && total_rank <= 64;
    // two to eight rows: the integer matrix-core kernel over the stacked rows, where it is the faster one
    const bool stacked_rows = !stacked && batch >= 2 && batch <= 8 && mv.count > 1 && ctx->gemv_i8 &&
                              (ctx->gemv_i8 == 2 || (k <= 2048 && mv.begin[mv.count] <= 4096)) &&
                              gemv_i8_multi_serves(mv, k, batch, ctx->cu_count);
    if (with_lora && !stacked && !stacked_rows) {
        // projection by projection: those that go to the few-token GEMM get their A . x there
        for (uint32_t i = 0, v = 0; i < count; ++i) {
            if (proj[i].n == 0) continue;
            if (ep[i].rank && gemv_takes_few_token_gemm(ctx, proj[i].n, k, batch) && gemm_skinny_computes_t(ep[i].rank, batch, proj[i].n)) {
                ep[i].a = proj[i].lora->a_packed;
                av.rank[v] = 0;
                --with_lora;
            }
            ++v;
        }
    }
    // ... and computes every A_v . x in producer workgroups of its own where CUs are left idle for them
    const bool rows_in_launch = stacked_rows && with_lora && ctx->lora_in_kernel &&
                                gemv_i8_lora_in_launch(mv.begin[mv.count], k, batch, total_rank, ctx->cu_count);
    if (with_lora) {  // the A . x buffer and the hand-over words belong to the context
        int rc = enter_shared_state(ctx, s);
        if (rc) return rc;
        if (!in_launch && !rows_in_launch) {
            launch_lora_a_views(av, k, x_dev, k, batch, s);  // every adapter's A . x in one launch
            ctx->counters.lora_a++;
        }
    }
    if (stacked_rows) {
        LoraEpilogue hand{};
        if (rows_in_launch) {
            hand.rank = total_rank;
            hand.slots = ctx->lora_slots_rows;
            hand.sync = ctx->lora_sync;
            hand.spin_limit = ctx->lora_spin_limit;
        }
        launch_gemv_i8_multi(mv, k, x_dev, k, batch, ctx->cu_count, rows_in_launch ? &hand : nullptr, s);
        ctx->counters.gemv_multi++;
    } else if (stacked) {
        LoraEpilogue hand{};
        if (in_launch) {
            hand.rank = total_rank;
            hand.slots = reinterpret_cast<unsigned long long*>(ctx->lora_sync + 64);
            hand.sync = ctx->lora_sync;
            hand.spin_limit = ctx->lora_spin_limit;
        }
        launch_gemv_multi(mv, k, x_dev, in_launch ? &hand : nullptr, s);
        ctx->counters.gemv_multi++;
    } else {
        // several rows (or a shape the stacked launch does not take): each projection through lq4_gemv's routing
        bool x_packed = false;  // the few-token GEMM's packed activations serve every projection that takes it
        for (uint32_t i = 0; i < count; ++i) {
            if (proj[i].n == 0) continue;
            int rc = gemv_dispatch(ctx, wp[i], proj[i].n, k, x_dev, batch, proj[i].y_dev, ep[i], s, &x_packed);
            if (rc) return rc;
        }
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_lora_apply(lq4_ctx* ctx, const lq4_lora* lora, float lora_scale, const void* x_dev, int x_dtype,
                   uint32_t rows, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (!lora || rows == 0) return LQ4_OK;  // no adapter for this projection: no-op
    if (!x_dev || !y_dev) return fail(LQ4_E_INVALID, "x/y device pointer is null");
    if (x_dtype != LQ4_F32 && x_dtype != LQ4_F16) return fail(LQ4_E_INVALID, "x_dtype must be LQ4_F32 or LQ4_F16");
    if (rows > kLoraTRows) return fail(LQ4_E_UNSUPPORTED, "LoRA call limited to %u rows, got %u", kLoraTRows, rows);
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    {
        const int rc = enter_shared_state(ctx, s);
        if (rc) return rc;
    }
    launch_lora_a(lora->a, lora->is_f16, lora->rank, lora->d_in, x_dev, x_dtype == LQ4_F16, lora->d_in, rows,
                  ctx->lora_t, s);
    launch_lora_b_accum(lora->b, lora->is_f16, lora->rank, lora->d_out, ctx->lora_t, lora_scale, rows, y_dev,
                        lora->d_out, s);
    ctx->counters.lora_a++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

// Called by every entry point that touches the context's shared state, before it launches anything (the
// context's device is current).  A call on another stream than the last one: that stream waits for an event
// recorded on the last one now, i.e. for everything queued there so far.  No host stall, and legal while either
// stream is being captured (the dependency then becomes part of the capture, as any cross-stream one does).
static int enter_shared_state(lq4_ctx* ctx, hipStream_t stream) {
    if (ctx->state_stream_known && ctx->state_stream != stream) {
        hipError_t e = hipEventRecord(ctx->state_event, ctx->state_stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(stream, ctx->state_event, 0);
        if (e != hipSuccess) {
            // (the previous stream may have been destroyed since: then the device is the only thing left to wait for)
            (void)hipGetLastError();
            hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
            if (cap != hipStreamCaptureStatusNone)
                return fail(LQ4_E_HIP, "cannot order this call behind the context's previous stream: %s", hipGetErrorString(e));
            LQ4_HIP(hipDeviceSynchronize());
        }
    }
    ctx->state_stream = stream;
    ctx->state_stream_known = true;
    return LQ4_OK;
}

// Grows one of the context's scratch buffers to `bytes`.  The outgrown buffer is kept until the
// context is destroyed: launches already queued, and launches captured into a graph, carry its
// address.  Nothing may be allocated while the stream is capturing: the call then fails and names
// lq4_ctx_reserve_scratch.  Steady-state calls reuse the buffer.
static int grow_scratch(lq4_ctx* ctx, uint8_t** buf, size_t* have, size_t bytes, hipStream_t stream, bool zero) {
    {
        const int rc = enter_shared_state(ctx, stream);
        if (rc) return rc;
    }
    if (bytes <= *have) return LQ4_OK;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) (void)hipGetLastError();
    if (cap != hipStreamCaptureStatusNone)
        return fail(LQ4_E_UNSUPPORTED,
                    "library scratch must grow from %zu to %zu bytes but the stream is capturing; run the shape once, or "
                    "call lq4_ctx_reserve_scratch, before the capture", *have, bytes);
    bytes = (bytes + (1u << 20) - 1) >> 20 << 20;
    uint8_t* fresh = nullptr;
    LQ4_HIP(hipMalloc(reinterpret_cast<void**>(&fresh), bytes));
    if (zero) {
        const hipError_t e = hipMemset(fresh, 0, bytes);
        if (e != hipSuccess) {
            (void)hipFree(fresh);
            return fail(LQ4_E_HIP, "hipMemset(scratch): %s", hipGetErrorString(e));
        }
    }
    if (*buf) ctx->retired.push_back(*buf);
    *buf = fresh;
    *have = bytes;
    return LQ4_OK;
}

static int ensure_scratch(lq4_ctx* ctx, size_t bytes, hipStream_t stream) {
    return grow_scratch(ctx, &ctx->moe_scratch, &ctx->moe_scratch_bytes, bytes, stream, false);
}

int lq4_ctx_reserve_scratch(lq4_ctx* ctx, size_t bytes) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    DeviceGuard g(ctx->device);
    const hipStream_t was = ctx->state_stream;  // (no launch: the stream of the last one stays)
    const bool known = ctx->state_stream_known;
    ctx->state_stream_known = false;
    // every growable buffer: which one an entry point uses is the library's business, not the caller's
    int rc = ensure_scratch(ctx, bytes, nullptr);
    if (!rc) rc = grow_scratch(ctx, &ctx->shared_scratch, &ctx->shared_scratch_bytes, bytes, nullptr, false);
    if (!rc) rc = grow_scratch(ctx, &ctx->chain_scratch, &ctx->chain_scratch_bytes, bytes, nullptr, false);
    ctx->state_stream = was;
    ctx->state_stream_known = known;
    return rc;
}

int lq4_gemm(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
             const void* x_dev, int x_dtype, uint32_t m, float* y_dev, const lq4_lora* lora,
             float lora_scale, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (m == 0 || n == 0) return LQ4_OK;
    if (x_dtype != LQ4_F32 && x_dtype != LQ4_F16) return fail(LQ4_E_INVALID, "x_dtype must be LQ4_F32 or LQ4_F16");
    if (x_dtype == LQ4_F32 && m <= kMaxGemvBatch)
        return lq4_gemv(ctx, w, w_extra_offset, n, k, static_cast<const float*>(x_dev), m, y_dev, lora, lora_scale, stream);
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    if (!x_dev || !y_dev) return fail(LQ4_E_INVALID, "x/y device pointer is null");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    LoraEpilogue ep;
    rc = resolve_lora(ctx, lora, lora_scale, n, k, m, &ep);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (ep.rank) {  // the A.x buffer (and, for one token, the hand-over words) belong to the context
        rc = enter_shared_state(ctx, s);
        if (rc) return rc;
    }
    if (ep.rank && gemm_takes_few_token_kernel(n, k, m, x_dtype == LQ4_F16, ctx->gemm_kernel) && gemm_skinny_computes_t(ep.rank, m, n)) {
        ep.a = lora->a_packed;  // the few-token GEMM computes A.X for its token tile itself
    } else if (ep.rank) {
        launch_lora_a(lora->a, lora->is_f16, lora->rank, k, x_dev, x_dtype == LQ4_F16, k, m, ctx->lora_t, s);
        ctx->counters.lora_a++;
    }
    // shapes with too few tiles run as K slices into scratch partials, summed by a second kernel
    const size_t scratch_bytes = gemm_scratch_floats(n, k, m, x_dtype == LQ4_F16, ep.rank != 0, ctx->gemm_kernel) * sizeof(float);
    if (scratch_bytes) {
        rc = ensure_scratch(ctx, scratch_bytes, static_cast<hipStream_t>(stream));
        if (rc) return rc;
    }
    launch_gemm(wp, n, k, x_dev, x_dtype == LQ4_F16, m, y_dev, ep,
                scratch_bytes ? reinterpret_cast<float*>(ctx->moe_scratch) : nullptr, ctx->gemm_kernel, s);
    ctx->counters.gemm++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_moe_route(lq4_ctx* ctx, const float* logits_dev, uint32_t tokens, uint32_t num_experts,
                  uint32_t top_k, int32_t* ids_dev, float* weights_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (tokens == 0) return LQ4_OK;
    if (!logits_dev || !ids_dev || !weights_dev) return fail(LQ4_E_INVALID, "null device pointer");
    if (top_k == 0 || top_k > 16 || top_k > num_experts)
        return fail(LQ4_E_INVALID, "top_k must be in 1..min(16, num_experts), got %u", top_k);
    if (num_experts > 1024) return fail(LQ4_E_INVALID, "num_experts %u above 1024", num_experts);
    DeviceGuard g(ctx->device);
    launch_moe_route(logits_dev, tokens, num_experts, top_k, ids_dev, weights_dev, static_cast<hipStream_t>(stream));
    ctx->counters.moe_route++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

// Scratch of the grouped expert kernels for `pairs` (token, slot) pairs over `experts` experts.
static int grouped_scratch(lq4_ctx* ctx, uint32_t experts, size_t pairs, uint32_t inter, uint32_t hidden,
                           hipStream_t stream, MoeScratch* s) {
    auto up256 = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t off_counts = 0;
    const size_t off_offsets = off_counts + up256(sizeof(int32_t) * experts);
    const size_t off_order = off_offsets + up256(sizeof(int32_t) * (experts + 1));
    const size_t off_h = off_order + up256(sizeof(int32_t) * pairs);
    const size_t off_o = off_h + up256(sizeof(float) * pairs * inter);
    const size_t total = off_o + up256(sizeof(float) * pairs * hidden);
    const int rc = ensure_scratch(ctx, total, stream);
    if (rc) return rc;
    s->counts = reinterpret_cast<int32_t*>(ctx->moe_scratch + off_counts);
    s->offsets = reinterpret_cast<int32_t*>(ctx->moe_scratch + off_offsets);
    s->order = reinterpret_cast<int32_t*>(ctx->moe_scratch + off_order);
    s->h = reinterpret_cast<float*>(ctx->moe_scratch + off_h);
    s->o = reinterpret_cast<float*>(ctx->moe_scratch + off_o);
    return LQ4_OK;
}

int lq4_moe_grouped_gemv(lq4_ctx* ctx, const lq4_weight* gate_up, const lq4_weight* down,
                         uint32_t num_experts, uint32_t inter, uint32_t hidden, const float* x_dev,
                         uint32_t tokens, const int32_t* ids_dev, const float* weights_dev,
                         uint32_t top_k, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (tokens == 0 || hidden == 0) return LQ4_OK;
    if (!x_dev || !ids_dev || !weights_dev || !y_dev) return fail(LQ4_E_INVALID, "null device pointer");
    if (num_experts == 0 || num_experts > 1024) return fail(LQ4_E_INVALID, "num_experts must be in 1..1024");
    if (top_k == 0 || static_cast<uint64_t>(tokens) * top_k > 4096)
        return fail(LQ4_E_INVALID, "tokens*top_k must be in 1..4096");
    if (inter == 0 || inter % kBlockWeights)
        return fail(LQ4_E_INVALID, "expert intermediate size must be a non-zero multiple of 32, got %u", inter);
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    const uint8_t *gu, *dn;
    const uint64_t gu_rows = static_cast<uint64_t>(num_experts) * 2 * inter;
    const uint64_t dn_rows = static_cast<uint64_t>(num_experts) * hidden;
    if (gu_rows > UINT32_MAX || dn_rows > UINT32_MAX) return fail(LQ4_E_INVALID, "expert tensor too large");
    int rc = resolve_weight(gate_up, 0, static_cast<uint32_t>(gu_rows), hidden, &gu);
    if (rc) return rc;
    rc = resolve_weight(down, 0, static_cast<uint32_t>(dn_rows), inter, &dn);
    if (rc) return rc;

    DeviceGuard g(ctx->device);
    // A few tokens (decode): per-pair one-token GEMVs.  Pairs rarely share an expert then, and what is
    // read twice costs less than the grouped kernels' fixed parts.
    static const uint32_t b1_tokens = [] {
        const char* env = getenv("LQ4_MOE_B1_TOKENS");
        return env ? static_cast<uint32_t>(strtoul(env, nullptr, 10)) : kMoeB1MaxTokens;
    }();
    if (tokens <= b1_tokens && moe_b1_serves(inter, hidden, top_k)) {
        rc = ensure_scratch(ctx, moe_b1_scratch_bytes(tokens, top_k, inter), static_cast<hipStream_t>(stream));
        if (rc) return rc;
        launch_moe_b1(gu, dn, num_experts, inter, hidden, x_dev, tokens, ids_dev, weights_dev, top_k, y_dev,
                      reinterpret_cast<float*>(ctx->moe_scratch), nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, false,
                      static_cast<hipStream_t>(stream));
        ctx->counters.moe_gate_up++;
        ctx->counters.moe_down++;
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    MoeScratch s;
    rc = grouped_scratch(ctx, num_experts, static_cast<size_t>(tokens) * top_k, inter, hidden,
                         static_cast<hipStream_t>(stream), &s);
    if (rc) return rc;
    launch_moe_grouped(gu, dn, num_experts, inter, hidden, x_dev, tokens, ids_dev, weights_dev, top_k, y_dev, s,
                       static_cast<hipStream_t>(stream));
    ctx->counters.moe_gate_up++;
    ctx->counters.moe_down++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

namespace {

// Scratch of the shared expert for `tokens` rows: [gate||up | act | out | packed activations of the
// few-token kernel], then (lq4_moe_ffn) the routing tables.
struct SharedScratch {
    size_t gu, act, o, pack, ids, wts, total;
};

SharedScratch shared_scratch_layout(uint32_t tokens, uint32_t shared_inter, uint32_t hidden, uint32_t top_k) {
    auto up256 = [](size_t v) { return (v + 255) / 256 * 256; };
    SharedScratch l;
    l.gu = 0;
    l.act = l.gu + up256(sizeof(float) * tokens * 2 * shared_inter);
    l.o = l.act + up256(sizeof(float) * tokens * shared_inter);
    l.pack = l.o + up256(sizeof(float) * tokens * hidden);
    const uint32_t kmax = hidden > shared_inter ? hidden : shared_inter;
    l.ids = l.pack + up256(tokens <= kMaxGemvBatch ? gemm_skinny_scratch_bytes(kmax, tokens) : 0);
    l.wts = l.ids + up256(sizeof(int32_t) * tokens * (top_k + 1));  // (one more slot: the shared expert's)
    l.total = l.wts + up256(sizeof(float) * tokens * (top_k + 1));
    return l;
}

// W . x for up to kMaxGemvBatch rows with explicit scratch (the routing of lq4_gemv without LoRA).
void small_batch_gemv(lq4_ctx* ctx, const uint8_t* wp, uint32_t n, uint32_t k, const float* x, uint32_t rows, float* y,
                      uint8_t* pack, hipStream_t s) {
    const LoraEpilogue none{};
    const uint64_t weights = static_cast<uint64_t>(n) * k;
    const bool narrow = n <= 2048 && gemv_mfma_lds_bytes(k, rows < 8 ? rows : 8) <= 150 * 1024;
    if (rows >= 9 || (rows >= 5 && n < 8192 && !narrow && weights >= 6000000)) {
        launch_gemm_skinny(wp, n, k, x, 0, rows, y, none, pack, s);
        ctx->counters.gemm++;
    } else if (rows == 1) {
        plain_gemv_one_token(ctx, wp, n, k, x, y, s);
    } else {
        launch_gemv(wp, n, k, x, k, rows, y, n, none, s);
        ctx->counters.gemv++;
    }
}

// The shared expert's FFN into scratch `o` (everything but the gate and the add).
// Returns LQ4_OK with the result in `o`, 1 when the per-pair kernels did everything (gate and add onto y_accum
// included: pass y_accum and shared_gate_dev to allow that), or an error.
int shared_expert_ffn(lq4_ctx* ctx, const lq4_weight* gate_up, const lq4_weight* down, const uint8_t* gu,
                      const uint8_t* dn, uint32_t shared_inter, uint32_t hidden, const float* x_dev, uint32_t tokens,
                      uint8_t* base, const SharedScratch& l, hipStream_t s, const float* shared_gate_dev = nullptr,
                      float* y_accum = nullptr) {
    float* gu_out = reinterpret_cast<float*>(base + l.gu);
    float* act = reinterpret_cast<float*>(base + l.act);
    float* o = reinterpret_cast<float*>(base + l.o);
    const LoraEpilogue none{};
    static const uint32_t alone_tokens = [] {
        const char* env = getenv("LQ4_MOE_SHARED_B1_TOKENS");
        return env ? static_cast<uint32_t>(strtoul(env, nullptr, 10)) : kSharedB1MaxTokens;
    }();
    if (y_accum && tokens <= alone_tokens && moe_b1_serves(shared_inter, hidden, 1)) {
        // a few tokens: the per-pair kernels with the shared expert as their only slot (its 2 MB are read
        // once from memory and then out of the caches), gate and add inside: two launches
        int rc = ensure_scratch(ctx, moe_b1_scratch_bytes(tokens, 1, shared_inter), s);
        if (rc) return rc;
        launch_moe_b1(gu, dn, 1, shared_inter, hidden, x_dev, tokens, nullptr, nullptr, 0, y_accum,
                      reinterpret_cast<float*>(ctx->moe_scratch), gu, dn, shared_gate_dev, nullptr, nullptr, nullptr, true, s);
        ctx->counters.moe_gate_up++;
        ctx->counters.moe_down++;
        return 1;  // done, including the gate and the add
    }
    if (tokens == 1 && gemv_b1_lds_bytes(shared_inter) <= 128 * 1024) {
        // gate||up, then the down projection with silu(gate) * up computed as it stages its activations
        launch_gemv(gu, 2 * shared_inter, hidden, x_dev, hidden, 1, gu_out, 2 * shared_inter, none, s);
        GemvFusion gf{};
        gf.prologue = GemvFusion::kSiluMul;
        gf.epilogue = GemvFusion::kStore;
        launch_gemv_b1_fused(dn, hidden, shared_inter, gu_out, o, none, gf, s);
        ctx->counters.gemv++;
        ctx->counters.gemv_fused++;
    } else if (tokens <= kMaxGemvBatch) {
        small_batch_gemv(ctx, gu, 2 * shared_inter, hidden, x_dev, tokens, gu_out, base + l.pack, s);
        launch_silu_mul(gu_out, shared_inter, tokens, act, shared_inter, s);
        ctx->counters.elementwise++;
        small_batch_gemv(ctx, dn, hidden, shared_inter, act, tokens, o, base + l.pack, s);
    } else {
        int rc = lq4_gemm(ctx, gate_up, 0, 2 * shared_inter, hidden, x_dev, LQ4_F32, tokens, gu_out, nullptr, 0.0f, s);
        if (rc) return rc;
        launch_silu_mul(gu_out, shared_inter, tokens, act, shared_inter, s);
        ctx->counters.elementwise++;
        rc = lq4_gemm(ctx, down, 0, hidden, shared_inter, act, LQ4_F32, tokens, o, nullptr, 0.0f, s);
        if (rc) return rc;
    }
    return LQ4_OK;
}

int check_shared_expert_args(const lq4_weight* gate_up, const lq4_weight* down, const float* shared_gate_dev,
                             uint32_t shared_inter, uint32_t hidden, const float* x_dev, const float* y_dev,
                             const uint8_t** gu, const uint8_t** dn) {
    if (!x_dev || !y_dev || !shared_gate_dev) return fail(LQ4_E_INVALID, "null device pointer");
    if (shared_inter == 0 || shared_inter % kBlockWeights)
        return fail(LQ4_E_INVALID, "shared expert intermediate size must be a non-zero multiple of 32, got %u", shared_inter);
    if (shared_inter > UINT32_MAX / 2) return fail(LQ4_E_INVALID, "shared expert intermediate size too large");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    int rc = resolve_weight(gate_up, 0, 2 * shared_inter, hidden, gu);
    if (rc) return rc;
    return resolve_weight(down, 0, hidden, shared_inter, dn);
}

}  // namespace

int lq4_moe_shared_expert(lq4_ctx* ctx, const lq4_weight* gate_up, const lq4_weight* down,
                          const float* shared_gate_dev, uint32_t shared_inter, uint32_t hidden, const float* x_dev,
                          uint32_t tokens, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (tokens == 0 || hidden == 0) return LQ4_OK;
    const uint8_t *gu, *dn;
    int rc = check_shared_expert_args(gate_up, down, shared_gate_dev, shared_inter, hidden, x_dev, y_dev, &gu, &dn);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    const SharedScratch l = shared_scratch_layout(tokens, shared_inter, hidden, 0);
    rc = grow_scratch(ctx, &ctx->shared_scratch, &ctx->shared_scratch_bytes, l.total, s, false);
    if (rc) return rc;
    rc = shared_expert_ffn(ctx, gate_up, down, gu, dn, shared_inter, hidden, x_dev, tokens, ctx->shared_scratch, l, s,
                           shared_gate_dev, y_dev);
    if (rc == 1) {
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    if (rc) return rc;
    launch_moe_shared_gate_add(x_dev, shared_gate_dev, reinterpret_cast<const float*>(ctx->shared_scratch + l.o), hidden,
                               tokens, y_dev, s);
    ctx->counters.elementwise++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_moe_ffn(lq4_ctx* ctx, const float* router_logits_dev, const lq4_weight* gate_up, const lq4_weight* down,
                uint32_t num_experts, uint32_t top_k, uint32_t inter, const lq4_weight* shared_gate_up,
                const lq4_weight* shared_down, const float* shared_gate_dev, uint32_t shared_inter, uint32_t hidden,
                const float* x_dev, uint32_t tokens, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (tokens == 0 || hidden == 0) return LQ4_OK;
    if (!router_logits_dev) return fail(LQ4_E_INVALID, "router logits pointer is null");
    if (top_k == 0 || top_k > 16 || top_k > num_experts)
        return fail(LQ4_E_INVALID, "top_k must be in 1..min(16, num_experts), got %u", top_k);
    if (static_cast<uint64_t>(tokens) * top_k > 4096) return fail(LQ4_E_INVALID, "tokens*top_k must be in 1..4096");
    const uint8_t *gu, *dn;
    int rc = check_shared_expert_args(shared_gate_up, shared_down, shared_gate_dev, shared_inter, hidden, x_dev, y_dev, &gu, &dn);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    const SharedScratch l = shared_scratch_layout(tokens, shared_inter, hidden, top_k);
    rc = grow_scratch(ctx, &ctx->shared_scratch, &ctx->shared_scratch_bytes, l.total, s, false);
    if (rc) return rc;
    uint8_t* base = ctx->shared_scratch;
    int32_t* ids = reinterpret_cast<int32_t*>(base + l.ids);
    float* wts = reinterpret_cast<float*>(base + l.wts);
    // A few tokens, shared expert as wide as the routed ones: it rides along as one more slot of the
    // per-pair kernels (route, gate||up, down: three launches for the whole layer).
    const uint8_t *rgu, *rdn;
    static const uint32_t b1_tokens = [] {
        const char* env = getenv("LQ4_MOE_B1_TOKENS");
        return env ? static_cast<uint32_t>(strtoul(env, nullptr, 10)) : kMoeB1MaxTokens;
    }();
    if (tokens <= b1_tokens && shared_inter == inter && inter % kBlockWeights == 0 && moe_b1_serves(inter, hidden, top_k + 1) &&
        num_experts <= 1024 && static_cast<uint64_t>(num_experts) * 2 * inter <= UINT32_MAX &&
        static_cast<uint64_t>(num_experts) * hidden <= UINT32_MAX) {
        rc = resolve_weight(gate_up, 0, num_experts * 2 * inter, hidden, &rgu);
        if (rc) return rc;
        rc = resolve_weight(down, 0, num_experts * hidden, inter, &rdn);
        if (rc) return rc;
        // up to 256 experts the gate||up launch routes as well: two launches for the layer
        const bool route_inside = num_experts <= 256;
        if (!route_inside) {
            rc = lq4_moe_route(ctx, router_logits_dev, tokens, num_experts, top_k, ids, wts, stream);
            if (rc) return rc;
        }
        rc = ensure_scratch(ctx, moe_b1_scratch_bytes(tokens, top_k + 1, inter), s);
        if (rc) return rc;
        launch_moe_b1(rgu, rdn, num_experts, inter, hidden, x_dev, tokens, ids, wts, top_k, y_dev,
                      reinterpret_cast<float*>(ctx->moe_scratch), gu, dn, shared_gate_dev,
                      route_inside ? router_logits_dev : nullptr, ids, wts, false, s);
        ctx->counters.moe_gate_up++;
        ctx->counters.moe_down++;
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    // More tokens, shared expert as wide as the routed ones: it rides along in the grouped kernels as expert
    // `num_experts`, chosen by every token in slot `top_k` with the sigmoid gate as its weight (the router
    // launch computes it): route, gate||up, down, combine, and none of the shared expert's own launches.
    // Whole layer, config 4's shapes, against the shared expert's own launches after the routed experts (16 / 64 /
    // 128 / 256 / 512 tokens): 61.8 / 100.2 / 152.3 / 270.6 / 455.6 -> 43.6 / 95.1 / 147.1 / 251.4 / 457.1 us.
    static const uint32_t grouped_tokens = [] {
        const char* env = getenv("LQ4_MOE_SHARED_GROUPED_TOKENS");
        return env ? static_cast<uint32_t>(strtoul(env, nullptr, 10)) : kMoeSharedGroupedMaxTokens;
    }();
    if (tokens > b1_tokens && tokens <= grouped_tokens && shared_inter == inter && num_experts < 1024 && moe_i8_serves(hidden) && moe_i8_serves(inter) &&
        static_cast<uint64_t>(num_experts) * 2 * inter <= UINT32_MAX &&
        static_cast<uint64_t>(num_experts) * hidden <= UINT32_MAX) {
        rc = resolve_weight(gate_up, 0, num_experts * 2 * inter, hidden, &rgu);
        if (rc) return rc;
        rc = resolve_weight(down, 0, num_experts * hidden, inter, &rdn);
        if (rc) return rc;
        MoeScratch ms;
        rc = grouped_scratch(ctx, num_experts + 1, static_cast<size_t>(tokens) * (top_k + 1), inter, hidden, s, &ms);
        if (rc) return rc;
        launch_moe_route(router_logits_dev, tokens, num_experts, top_k, ids, wts, s, x_dev, shared_gate_dev, hidden);
        ctx->counters.moe_route++;
        launch_moe_grouped(rgu, rdn, num_experts, inter, hidden, x_dev, tokens, ids, wts, top_k, y_dev, ms, s, gu, dn);
        ctx->counters.moe_gate_up++;
        ctx->counters.moe_down++;
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    // One stream: running the shared expert beside the routed experts on a second stream (forked and
    // joined with events) was measured slower, eagerly and in a captured graph alike (1 token 38.3 ->
    // 47.8 us, 16 tokens 68.0 -> 66.9 eager / 72.3 captured): each of these launches fills the GPU by
    // itself, and the cross-stream waits cost more than the overlap of their ramps returns.
    rc = lq4_moe_route(ctx, router_logits_dev, tokens, num_experts, top_k, ids, wts, stream);
    if (rc) return rc;
    rc = lq4_moe_grouped_gemv(ctx, gate_up, down, num_experts, inter, hidden, x_dev, tokens, ids, wts, top_k, y_dev, stream);
    if (rc) return rc;
    rc = shared_expert_ffn(ctx, shared_gate_up, shared_down, gu, dn, shared_inter, hidden, x_dev, tokens, base, l, s,
                           shared_gate_dev, y_dev);
    if (rc == 1) {
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    if (rc) return rc;
    launch_moe_shared_gate_add(x_dev, shared_gate_dev, reinterpret_cast<const float*>(base + l.o), hidden, tokens, y_dev, s);
    ctx->counters.elementwise++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_dequant(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                float* out_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (n == 0) return LQ4_OK;
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    if (!out_dev || reinterpret_cast<uintptr_t>(out_dev) % 8) return fail(LQ4_E_INVALID, "out must be non-null and 8-byte aligned");
    DeviceGuard g(ctx->device);
    launch_dequant(wp, n, k, out_dev, static_cast<hipStream_t>(stream));
    ctx->counters.dequant++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_probe_read_config(lq4_ctx* ctx, const void* p_dev, size_t nbytes, uint32_t workgroups, uint32_t bytes_in_flight,
                          int strided, int nontemporal, void* stream) {
    if (!ctx || !p_dev) return fail(LQ4_E_INVALID, "null argument");
    if (reinterpret_cast<uintptr_t>(p_dev) % 16) return fail(LQ4_E_INVALID, "buffer must be 16-byte aligned");
    if (workgroups > 65536) return fail(LQ4_E_INVALID, "at most 65536 workgroups");
    DeviceGuard g(ctx->device);
    if (!launch_probe_read(p_dev, nbytes, workgroups, bytes_in_flight, strided != 0, nontemporal != 0,
                           reinterpret_cast<uint32_t*>(ctx->lora_t), static_cast<hipStream_t>(stream)))
        return fail(LQ4_E_INVALID, "bytes_in_flight must be 64, 128 or 256, got %u", bytes_in_flight);
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_probe_read(lq4_ctx* ctx, const void* p_dev, size_t nbytes, void* stream) {
    // the configuration that won the sweep at every size from 8 MB to 1 GB
    return lq4_probe_read_config(ctx, p_dev, nbytes, 0, 128, 1, 1, stream);
}

int lq4_topk(lq4_ctx* ctx, const float* logits_dev, uint32_t n, uint32_t top_k, float* out_logits_dev,
             uint32_t* out_ids_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (top_k == 0) return LQ4_OK;
    if (!logits_dev || !out_logits_dev || !out_ids_dev) return fail(LQ4_E_INVALID, "null device pointer");
    if (top_k > LQ4_MAX_TOP_K) return fail(LQ4_E_INVALID, "top_k %u above %d", top_k, LQ4_MAX_TOP_K);
    if (n == 0) return fail(LQ4_E_INVALID, "no logits to select from");
    DeviceGuard g(ctx->device);
    const int rc = ensure_scratch(ctx, topk_scratch_bytes(n, top_k), static_cast<hipStream_t>(stream));
    if (rc) return rc;
    launch_topk(logits_dev, n, top_k, ctx->moe_scratch, ctx->topk_ticket, out_logits_dev, out_ids_dev,
                static_cast<hipStream_t>(stream));
    ctx->counters.topk++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

namespace {


// Scratch of one lm_head + top-k call: [vocab logits | maxima, candidates].
size_t lm_head_scratch_need(uint32_t vocab, uint32_t top_k) {
    const size_t logits_bytes = (static_cast<size_t>(vocab) * sizeof(float) + 255) / 256 * 256;
    return logits_bytes + topk_scratch_bytes(vocab, top_k);
}

int lm_head_topk_common(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t vocab, uint32_t k,
                        const float* x_dev, uint32_t top_k, float* out_logits_dev, uint32_t* out_ids_dev, void* stream,
                        bool static_scratch) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (top_k == 0) return LQ4_OK;
    if (vocab == 0) return fail(LQ4_E_INVALID, "empty vocabulary");
    if (top_k > LQ4_MAX_TOP_K) return fail(LQ4_E_INVALID, "top_k %u above %d", top_k, LQ4_MAX_TOP_K);
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, vocab, k, &wp);
    if (rc) return rc;
    if (!x_dev || !out_logits_dev || !out_ids_dev) return fail(LQ4_E_INVALID, "null device pointer");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    const size_t need = lm_head_scratch_need(vocab, top_k);
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    uint8_t* base;
    if (static_scratch) {
        if (need > kStaticScratchBytes)
            return fail(LQ4_E_UNSUPPORTED,
                        "lq4_lm_head_topk_static: vocab %u with top_k %u needs %zu bytes of scratch, the static buffer holds %zu; "
                        "use lq4_lm_head_topk", vocab, top_k, need, kStaticScratchBytes);
        base = ctx->static_scratch;
        rc = enter_shared_state(ctx, s);  // the static array and the ticket word are shared like the scratch
        if (rc) return rc;
    } else {
        rc = ensure_scratch(ctx, need, s);
        if (rc) return rc;
        base = ctx->moe_scratch;
    }
    const size_t logits_bytes = (static_cast<size_t>(vocab) * sizeof(float) + 255) / 256 * 256;
    float* logits = reinterpret_cast<float*>(base);
    plain_gemv_one_token(ctx, wp, vocab, k, x_dev, logits, s);
    launch_topk(logits, vocab, top_k, base + logits_bytes, ctx->topk_ticket, out_logits_dev, out_ids_dev, s);
    ctx->counters.topk++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

}  // namespace

int lq4_lm_head_topk(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t vocab, uint32_t k,
                     const float* x_dev, uint32_t top_k, float* out_logits_dev, uint32_t* out_ids_dev,
                     void* stream) {
    return lm_head_topk_common(ctx, w, w_extra_offset, vocab, k, x_dev, top_k, out_logits_dev, out_ids_dev, stream, false);
}

// The same call with its scratch in the library's static array: allocates nothing.
int lq4_lm_head_topk_static(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t vocab, uint32_t k,
                            const float* x_dev, uint32_t top_k, float* out_logits_dev, uint32_t* out_ids_dev,
                            void* stream) {
    return lm_head_topk_common(ctx, w, w_extra_offset, vocab, k, x_dev, top_k, out_logits_dev, out_ids_dev, stream, true);
}

int lq4_residual_add_rmsnorm(lq4_ctx* ctx, const float* base_dev, const float* delta_dev, const float* gamma_dev,
                             uint32_t hidden, uint32_t rows, float eps, float* residual_out_dev,
                             float* normed_out_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (rows == 0 || hidden == 0) return LQ4_OK;
    if (!base_dev || !gamma_dev || !normed_out_dev) return fail(LQ4_E_INVALID, "base, gamma or normed_out is null");
    DeviceGuard g(ctx->device);
    launch_residual_add_norm(base_dev, delta_dev, gamma_dev, hidden, rows, eps, residual_out_dev, normed_out_dev,
                             static_cast<hipStream_t>(stream));
    ctx->counters.elementwise++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_silu_mul(lq4_ctx* ctx, const float* gate_up_dev, uint32_t count, uint32_t rows, float* out_dev,
                 uint32_t out_stride, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (rows == 0 || count == 0) return LQ4_OK;
    if (!gate_up_dev || !out_dev) return fail(LQ4_E_INVALID, "gate_up or out is null");
    if (out_stride < count) return fail(LQ4_E_INVALID, "out_stride %u below count %u", out_stride, count);
    if (rows > 65535) return fail(LQ4_E_UNSUPPORTED, "silu_mul limited to 65535 rows, got %u", rows);
    DeviceGuard g(ctx->device);
    launch_silu_mul(gate_up_dev, count, rows, out_dev, out_stride, static_cast<hipStream_t>(stream));
    ctx->counters.elementwise++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_add_and_copy(lq4_ctx* ctx, const float* src_dev, float* residual_dev, float* dst_dev, size_t count,
                     void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (count == 0) return LQ4_OK;
    if (!src_dev || !residual_dev) return fail(LQ4_E_INVALID, "src or residual is null");
    DeviceGuard g(ctx->device);
    launch_add_and_copy(src_dev, residual_dev, dst_dev, count, static_cast<hipStream_t>(stream));
    ctx->counters.elementwise++;
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

static bool ranges_overlap(const void* a, const void* b, size_t bytes) {
    const uintptr_t pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + bytes && pb < pa + bytes;
}

int lq4_gemv_fused(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                   const float* x_dev, float* y_dev, const lq4_gemv_fusion* fusion, const lq4_lora* lora,
                   float lora_scale, void* stream) {
    if (!fusion || (fusion->prologue == LQ4_PRO_NONE && fusion->epilogue == LQ4_EPI_NONE))
        return lq4_gemv(ctx, w, w_extra_offset, n, k, x_dev, 1, y_dev, lora, lora_scale, stream);
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (n == 0) return LQ4_OK;
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    const lq4_gemv_fusion& f = *fusion;
    const size_t kbytes = static_cast<size_t>(k) * sizeof(float);
    auto misaligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
    switch (f.prologue) {
        case LQ4_PRO_NONE:
        case LQ4_PRO_SILU_MUL:
            if (!x_dev) return fail(LQ4_E_INVALID, "x device pointer is null");
            if (misaligned(x_dev)) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
            break;
        case LQ4_PRO_ADD_RMSNORM:
            if (!f.base || !f.gamma) return fail(LQ4_E_INVALID, "fusion.base or fusion.gamma is null");
            if (misaligned(f.base) || misaligned(f.gamma) || (f.delta && misaligned(f.delta)) ||
                (f.residual_out && misaligned(f.residual_out)))
                return fail(LQ4_E_INVALID, "fusion.base, delta, gamma and residual_out must be 16-byte aligned");
            if (f.residual_out && (ranges_overlap(f.residual_out, f.base, kbytes) ||
                                   (f.delta && ranges_overlap(f.residual_out, f.delta, kbytes))))
                return fail(LQ4_E_INVALID, "fusion.residual_out must not overlap fusion.base or fusion.delta");
            break;
        default:
            return fail(LQ4_E_INVALID, "unknown fusion.prologue %d", f.prologue);
    }
    if (f.epilogue == LQ4_EPI_ADD_RESIDUAL) {
        if (!f.residual) return fail(LQ4_E_INVALID, "fusion.residual is null");
        if (reinterpret_cast<uintptr_t>(f.residual) % 4 || reinterpret_cast<uintptr_t>(f.copy_dst) % 4)
            return fail(LQ4_E_INVALID, "fusion.residual and copy_dst must be 4-byte aligned");
    } else if (f.epilogue == LQ4_EPI_NONE) {
        if (!y_dev) return fail(LQ4_E_INVALID, "y device pointer is null");
    } else if (f.epilogue == LQ4_EPI_SILU_MUL_PAIRS) {
        if (!y_dev) return fail(LQ4_E_INVALID, "y device pointer is null");
        if (n % 2) return fail(LQ4_E_INVALID, "LQ4_EPI_SILU_MUL_PAIRS needs an even number of rows, got %u", n);
    } else {
        return fail(LQ4_E_INVALID, "unknown fusion.epilogue %d", f.epilogue);
    }
    if (y_dev && reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    LoraEpilogue ep;
    rc = resolve_lora(ctx, lora, lora_scale, n, k, 1, &ep);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (ep.rank) {  // the A.x buffer (and, for one token, the hand-over words) belong to the context
        rc = enter_shared_state(ctx, s);
        if (rc) return rc;
    }

    const bool pairs = f.epilogue == LQ4_EPI_SILU_MUL_PAIRS;
    const bool fused_ok = gemv_b1_lds_bytes(k) <= 128 * 1024 && !(ep.rank && f.prologue != LQ4_PRO_NONE) &&
                          !(pairs && (ep.rank || !gemv_b1_pairs_served(n, k)));
    if (fused_ok) {
        if (ep.rank) {
            launch_lora_a(lora->a, lora->is_f16, lora->rank, k, x_dev, 0, k, 1, ctx->lora_t, s);
            ctx->counters.lora_a++;
        }
        GemvFusion gf;
        gf.prologue = f.prologue;
        gf.base = f.base;
        gf.delta = f.delta;
        gf.gamma = f.gamma;
        gf.eps = f.eps;
        gf.residual_out = f.residual_out;
        gf.epilogue = f.epilogue;
        gf.residual = f.residual;
        gf.copy_dst = f.copy_dst;
        launch_gemv_b1_fused(wp, n, k, x_dev, y_dev, ep, gf, s);
        ctx->counters.gemv_fused++;
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }

    // The same steps one by one: activations and (if the caller wants no y) the product in scratch.
    const size_t x_off = 0, y_off = (kbytes + 255) / 256 * 256;
    rc = ensure_scratch(ctx, y_off + static_cast<size_t>(n) * sizeof(float), static_cast<hipStream_t>(stream));
    if (rc) return rc;
    if (pairs) {  // the product [gate | up] in scratch, then silu(gate) * up into y
        const float* act_p = x_dev;
        float* xs_p = reinterpret_cast<float*>(ctx->moe_scratch + x_off);
        if (f.prologue == LQ4_PRO_ADD_RMSNORM) {
            launch_residual_add_norm(f.base, f.delta, f.gamma, k, 1, f.eps, f.residual_out, xs_p, s);
            act_p = xs_p;
            ctx->counters.elementwise++;
        } else if (f.prologue == LQ4_PRO_SILU_MUL) {
            launch_silu_mul(x_dev, k, 1, xs_p, k, s);
            act_p = xs_p;
            ctx->counters.elementwise++;
        }
        if (ep.rank) {
            launch_lora_a(lora->a, lora->is_f16, lora->rank, k, act_p, 0, k, 1, ctx->lora_t, s);
            ctx->counters.lora_a++;
        }
        float* gu = reinterpret_cast<float*>(ctx->moe_scratch + y_off);
        launch_gemv(wp, n, k, act_p, k, 1, gu, n, ep, s);
        ctx->counters.gemv++;
        launch_silu_mul(gu, n / 2, 1, y_dev, n / 2, s);
        ctx->counters.elementwise++;
        LQ4_HIP(hipGetLastError());
        return LQ4_OK;
    }
    const float* act = x_dev;
    float* xs = reinterpret_cast<float*>(ctx->moe_scratch + x_off);
    if (f.prologue == LQ4_PRO_ADD_RMSNORM) {
        launch_residual_add_norm(f.base, f.delta, f.gamma, k, 1, f.eps, f.residual_out, xs, s);
        act = xs;
        ctx->counters.elementwise++;
    } else if (f.prologue == LQ4_PRO_SILU_MUL) {
        launch_silu_mul(x_dev, k, 1, xs, k, s);
        act = xs;
        ctx->counters.elementwise++;
    }
    if (ep.rank) {
        launch_lora_a(lora->a, lora->is_f16, lora->rank, k, act, 0, k, 1, ctx->lora_t, s);
        ctx->counters.lora_a++;
    }
    float* yo = y_dev ? y_dev : reinterpret_cast<float*>(ctx->moe_scratch + y_off);
    launch_gemv(wp, n, k, act, k, 1, yo, n, ep, s);
    ctx->counters.gemv++;
    if (f.epilogue == LQ4_EPI_ADD_RESIDUAL) {
        launch_add_and_copy(yo, f.residual, f.copy_dst, n, s);
        ctx->counters.elementwise++;
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_gemv_fused_batch(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                         const float* x_dev, uint32_t batch, float* y_dev, const lq4_gemv_fusion* fusion,
                         const lq4_lora* lora, float lora_scale, void* stream) {
    if (batch == 1) return lq4_gemv_fused(ctx, w, w_extra_offset, n, k, x_dev, y_dev, fusion, lora, lora_scale, stream);
    if (!fusion || (fusion->prologue == LQ4_PRO_NONE && fusion->epilogue == LQ4_EPI_NONE))
        return lq4_gemv(ctx, w, w_extra_offset, n, k, x_dev, batch, y_dev, lora, lora_scale, stream);
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (batch == 0 || n == 0) return LQ4_OK;
    if (batch > LQ4_MAX_GEMV_BATCH) return fail(LQ4_E_INVALID, "batch %u above %d", batch, LQ4_MAX_GEMV_BATCH);
    const uint8_t* wp;
    int rc = resolve_weight(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    const lq4_gemv_fusion& f = *fusion;
    const size_t in_bytes = static_cast<size_t>(batch) * k * sizeof(float);
    auto misaligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 != 0; };
    switch (f.prologue) {
        case LQ4_PRO_NONE:
        case LQ4_PRO_SILU_MUL:
            if (!x_dev) return fail(LQ4_E_INVALID, "x device pointer is null");
            if (misaligned(x_dev)) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
            break;
        case LQ4_PRO_ADD_RMSNORM:
            if (!f.base || !f.gamma) return fail(LQ4_E_INVALID, "fusion.base or fusion.gamma is null");
            if (misaligned(f.base) || misaligned(f.gamma) || (f.delta && misaligned(f.delta)) ||
                (f.residual_out && misaligned(f.residual_out)))
                return fail(LQ4_E_INVALID, "fusion.base, delta, gamma and residual_out must be 16-byte aligned");
            if (f.residual_out && (ranges_overlap(f.residual_out, f.base, in_bytes) ||
                                   (f.delta && ranges_overlap(f.residual_out, f.delta, in_bytes))))
                return fail(LQ4_E_INVALID, "fusion.residual_out must not overlap fusion.base or fusion.delta");
            break;
        default:
            return fail(LQ4_E_INVALID, "unknown fusion.prologue %d", f.prologue);
    }
    if (f.epilogue == LQ4_EPI_ADD_RESIDUAL) {
        if (!f.residual) return fail(LQ4_E_INVALID, "fusion.residual is null");
        if (reinterpret_cast<uintptr_t>(f.residual) % 4 || reinterpret_cast<uintptr_t>(f.copy_dst) % 4)
            return fail(LQ4_E_INVALID, "fusion.residual and copy_dst must be 4-byte aligned");
    } else if (f.epilogue == LQ4_EPI_NONE) {
        if (!y_dev) return fail(LQ4_E_INVALID, "y device pointer is null");
    } else {
        return fail(LQ4_E_INVALID, "unknown fusion.epilogue %d", f.epilogue);
    }
    if (y_dev && reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    LoraEpilogue ep;
    rc = resolve_lora(ctx, lora, lora_scale, n, k, batch, &ep);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (ep.rank) {  // the A.x buffer (and, for one token, the hand-over words) belong to the context
        rc = enter_shared_state(ctx, s);
        if (rc) return rc;
    }

    // Inside the launch every workgroup produces all rows' activations for itself: that pays while the
    // rows are small (one token always; more rows up to this many bytes of prologue input per workgroup:
    // the decode MLP of a 2048-wide model at 3 and 4 rows 21.2 / 22.1 -> 19.6 / 21.2 us, at 8 rows
    // 26.4 -> 32.7 us with everything inside).  Larger inputs run the prologue once, as its own launch, and
    // keep only the epilogue in the GEMV.  More than 8 rows are served by the few-token GEMM kernel,
    // which has no fused form: the steps run one by one.
    const size_t pro_bytes = f.prologue == LQ4_PRO_NONE ? 0 : in_bytes * (f.prologue == LQ4_PRO_SILU_MUL ? 2 : (f.delta ? 2 : 1));
    static const size_t pro_limit = [] {
        const char* env = getenv("LQ4_FUSED_PROLOGUE_BYTES");
        return env ? static_cast<size_t>(strtoull(env, nullptr, 10)) : kFusedPrologueBytes;
    }();
    if (!ep.rank && batch <= 8 && gemv_fused_batch_fits(k, batch)) {
        GemvFusion gf;
        const float* act_in = x_dev;
        int pro = f.prologue;
        if (pro_bytes > pro_limit) {
            rc = ensure_scratch(ctx, in_bytes, s);
            if (rc) return rc;
            float* xs = reinterpret_cast<float*>(ctx->moe_scratch);
            if (pro == LQ4_PRO_ADD_RMSNORM) launch_residual_add_norm(f.base, f.delta, f.gamma, k, batch, f.eps, f.residual_out, xs, s);
            else launch_silu_mul(x_dev, k, batch, xs, k, s);
            ctx->counters.elementwise++;
            act_in = xs;
            pro = LQ4_PRO_NONE;
        }
        gf.prologue = pro;
        gf.base = f.base;
        gf.delta = f.delta;
        gf.gamma = f.gamma;
        gf.eps = f.eps;
        gf.residual_out = f.residual_out;
        gf.epilogue = f.epilogue;
        gf.residual = f.residual;
        gf.copy_dst = f.copy_dst;
        if (launch_gemv_fused_batch(wp, n, k, act_in, batch, y_dev, gf, s)) {
            ctx->counters.gemv_fused++;
            LQ4_HIP(hipGetLastError());
            return LQ4_OK;
        }
    }

    // The same steps one by one: activations and (if the caller wants no y) the product in scratch (not
    // the scratch lq4_gemv itself may use for its few-token kernel).
    const size_t y_off = (in_bytes + 255) / 256 * 256;
    rc = grow_scratch(ctx, &ctx->shared_scratch, &ctx->shared_scratch_bytes,
                      y_off + static_cast<size_t>(batch) * n * sizeof(float), s, false);
    if (rc) return rc;
    const float* act = x_dev;
    float* xs = reinterpret_cast<float*>(ctx->shared_scratch);
    if (f.prologue == LQ4_PRO_ADD_RMSNORM) {
        launch_residual_add_norm(f.base, f.delta, f.gamma, k, batch, f.eps, f.residual_out, xs, s);
        act = xs;
        ctx->counters.elementwise++;
    } else if (f.prologue == LQ4_PRO_SILU_MUL) {
        launch_silu_mul(x_dev, k, batch, xs, k, s);
        act = xs;
        ctx->counters.elementwise++;
    }
    float* yo = y_dev ? y_dev : reinterpret_cast<float*>(ctx->shared_scratch + y_off);
    rc = lq4_gemv(ctx, w, w_extra_offset, n, k, act, batch, yo, lora, lora_scale, stream);
    if (rc) return rc;
    if (f.epilogue == LQ4_EPI_ADD_RESIDUAL) {
        launch_add_and_copy(yo, f.residual, f.copy_dst, static_cast<size_t>(batch) * n, s);
        ctx->counters.elementwise++;
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

// ---- a chain of batch-1 GEMVs --------------------------------------------------------------------
namespace {

inline size_t up256(size_t v) { return (v + 255) / 256 * 256; }

inline uint32_t chain_result_len(const lq4_chain_step& st) {
    return st.epilogue == LQ4_EPI_SILU_MUL_PAIRS ? st.n / 2 : st.n;
}

// The plain pointer a step's result is stored at for the caller (null: nowhere).
inline const float* chain_result_ptr(const lq4_chain_step& st) {
    return st.y_dev ? st.y_dev : st.epilogue == LQ4_EPI_ADD_RESIDUAL ? st.residual : nullptr;
}

int chain_validate(const lq4_chain_step* steps, uint32_t n_steps) {
    auto misaligned = [](const void* p, uintptr_t a) { return reinterpret_cast<uintptr_t>(p) % a != 0; };
    for (uint32_t j = 0; j < n_steps; ++j) {
        const lq4_chain_step& st = steps[j];
        if (st.n == 0) return fail(LQ4_E_INVALID, "chain step %u has no rows", j);
        const uint8_t* wp;
        const int rc = resolve_weight(st.w, st.w_extra_offset, st.n, st.k, &wp);
        if (rc) return rc;
        if (st.from_previous) {
            if (j == 0) return fail(LQ4_E_INVALID, "chain step 0 needs external activations");
            if (st.prologue != LQ4_PRO_NONE && st.prologue != LQ4_PRO_ADD_RMSNORM)
                return fail(LQ4_E_INVALID, "chain step %u: a step fed by the previous result takes LQ4_PRO_NONE or LQ4_PRO_ADD_RMSNORM", j);
            if (chain_result_len(steps[j - 1]) != st.k)
                return fail(LQ4_E_INVALID, "chain step %u: K = %u but the previous step yields %u values", j, st.k,
                            chain_result_len(steps[j - 1]));
            if (st.x_dev || st.delta)
                return fail(LQ4_E_INVALID, "chain step %u: from_previous puts the previous result in the place of x_dev / delta; leave both null", j);
        } else if (st.prologue == LQ4_PRO_NONE || st.prologue == LQ4_PRO_SILU_MUL) {
            if (!st.x_dev || misaligned(st.x_dev, 16)) return fail(LQ4_E_INVALID, "chain step %u: x must be non-null and 16-byte aligned", j);
        }
        switch (st.prologue) {
            case LQ4_PRO_NONE:
            case LQ4_PRO_SILU_MUL:
                break;
            case LQ4_PRO_ADD_RMSNORM: {
                if (!st.gamma || misaligned(st.gamma, 16)) return fail(LQ4_E_INVALID, "chain step %u: gamma must be non-null and 16-byte aligned", j);
                if (!st.from_previous && !st.base) return fail(LQ4_E_INVALID, "chain step %u: base is null", j);
                if (misaligned(st.base, 16) || misaligned(st.delta, 16) || misaligned(st.residual_out, 16))
                    return fail(LQ4_E_INVALID, "chain step %u: base, delta and residual_out must be 16-byte aligned", j);
                const size_t kb = static_cast<size_t>(st.k) * 4;
                if (st.residual_out && ((st.base && ranges_overlap(st.residual_out, st.base, kb)) ||
                                        (st.delta && ranges_overlap(st.residual_out, st.delta, kb))))
                    return fail(LQ4_E_INVALID, "chain step %u: residual_out must not overlap base or delta", j);
                break;
            }
            default:
                return fail(LQ4_E_INVALID, "chain step %u: unknown prologue %d", j, st.prologue);
        }
        switch (st.epilogue) {
            case LQ4_EPI_NONE:
                break;
            case LQ4_EPI_ADD_RESIDUAL:
                if (!st.residual || misaligned(st.residual, 16)) return fail(LQ4_E_INVALID, "chain step %u: residual must be non-null and 16-byte aligned", j);
                break;
            case LQ4_EPI_SILU_MUL_PAIRS:
                if (st.n % 2) return fail(LQ4_E_INVALID, "chain step %u: silu(gate) * up over row pairs needs an even N, got %u", j, st.n);
                break;
            default:
                return fail(LQ4_E_INVALID, "chain step %u: unknown epilogue %d", j, st.epilogue);
        }
        if (st.y_dev && misaligned(st.y_dev, 16)) return fail(LQ4_E_INVALID, "chain step %u: y must be 16-byte aligned", j);
        if (j + 1 == n_steps && !chain_result_ptr(st))
            return fail(LQ4_E_INVALID, "the last chain step has nowhere to put its result (y_dev is null)");
    }
    return LQ4_OK;
}

// Byte offsets, in the chain scratch, of every step's result vector, and the total.
struct ChainLayout {
    size_t result[LQ4_CHAIN_MAX_STEPS], total;
};
ChainLayout chain_scratch_layout(const lq4_chain_step* steps, uint32_t n_steps) {
    ChainLayout l;
    l.total = 0;
    for (uint32_t j = 0; j < n_steps; ++j) {
        l.result[j] = l.total;
        l.total += up256(static_cast<size_t>(steps[j].n) * 4);  // n, not n/2: a [gate | up] vector may be kept here
    }
    return l;
}

}  // namespace

int lq4_gemv_chain(lq4_ctx* ctx, const lq4_chain_step* steps, uint32_t n_steps, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (n_steps == 0) return LQ4_OK;
    if (!steps) return fail(LQ4_E_INVALID, "steps is null");
    if (n_steps > LQ4_CHAIN_MAX_STEPS) return fail(LQ4_E_INVALID, "a chain holds at most %d steps, got %u", LQ4_CHAIN_MAX_STEPS, n_steps);
    int rc = chain_validate(steps, n_steps);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    const ChainLayout lay = chain_scratch_layout(steps, n_steps);
    rc = grow_scratch(ctx, &ctx->chain_scratch, &ctx->chain_scratch_bytes, lay.total, s, false);
    if (rc) return rc;

    ctx->counters.gemv_chain++;

    // Step by step: every step is lq4_gemv_fused; results nobody asked for live in the chain scratch as
    // plain floats.  A step that ends in silu(gate) * up runs plain and the NEXT step takes gate || up
    // through its silu prologue (LQ4_PRO_SILU_MUL), which costs no launch; only when the caller wants the
    // product itself (y_dev), or nothing plain follows, does the stand-alone silu * up kernel run.
    const float* prev = nullptr;
    bool prev_is_gate_up = false;  // prev holds [gate | up] of the previous step, silu * up still to apply
    for (uint32_t j = 0; j < n_steps; ++j) {
        const lq4_chain_step& st = steps[j];
        float* spare = reinterpret_cast<float*>(ctx->chain_scratch + lay.result[j]);
        lq4_gemv_fusion f;
        std::memset(&f, 0, sizeof f);
        const float* x = st.x_dev;
        f.prologue = st.prologue;
        f.gamma = st.gamma;
        f.eps = st.eps;
        f.base = st.base;
        f.delta = st.delta;
        f.residual_out = st.residual_out;
        if (st.from_previous) {
            if (st.prologue != LQ4_PRO_ADD_RMSNORM) {
                x = prev;
                if (prev_is_gate_up) f.prologue = LQ4_PRO_SILU_MUL;
            } else if (st.base) {
                f.delta = prev;
            } else {
                f.base = prev;
            }
        }
        prev_is_gate_up = false;
        float* result;
        if (st.epilogue == LQ4_EPI_ADD_RESIDUAL) {
            f.epilogue = LQ4_EPI_ADD_RESIDUAL;
            f.residual = st.residual;
            f.copy_dst = st.y_dev;
            rc = lq4_gemv_fused(ctx, st.w, st.w_extra_offset, st.n, st.k, x, nullptr, &f, nullptr, 0.0f, stream);
            result = st.residual;
        } else if (st.epilogue == LQ4_EPI_SILU_MUL_PAIRS && gemv_b1_pairs_served(st.n, st.k) &&
                   gemv_b1_lds_bytes(st.k) <= 128 * 1024) {
            // the launch writes silu(gate) * up itself: no [gate | up] vector, no step after it
            f.epilogue = LQ4_EPI_SILU_MUL_PAIRS;
            result = st.y_dev ? st.y_dev : spare;
            rc = lq4_gemv_fused(ctx, st.w, st.w_extra_offset, st.n, st.k, x, result, &f, nullptr, 0.0f, stream);
        } else if (st.epilogue == LQ4_EPI_SILU_MUL_PAIRS) {
            f.epilogue = LQ4_EPI_NONE;
            rc = lq4_gemv_fused(ctx, st.w, st.w_extra_offset, st.n, st.k, x, spare, &f, nullptr, 0.0f, stream);
            const bool next_takes_it = !st.y_dev && j + 1 < n_steps && steps[j + 1].from_previous &&
                                       steps[j + 1].prologue == LQ4_PRO_NONE;
            if (next_takes_it) {
                result = spare;
                prev_is_gate_up = true;
            } else {
                result = st.y_dev ? st.y_dev : spare;  // in place: out[i] only depends on in[i] and in[i + n/2]
                if (!rc) {
                    launch_silu_mul(spare, st.n / 2, 1, result, st.n / 2, s);
                    ctx->counters.elementwise++;
                }
            }
        } else {
            f.epilogue = LQ4_EPI_NONE;
            result = st.y_dev ? st.y_dev : spare;
            rc = lq4_gemv_fused(ctx, st.w, st.w_extra_offset, st.n, st.k, x, result, &f, nullptr, 0.0f, stream);
        }
        if (rc) return rc;
        prev = result;
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_gemm_q8(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const void* x_dev, int x_dtype, uint32_t m, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (m == 0 || n == 0) return LQ4_OK;
    if (x_dtype != LQ4_F32 && x_dtype != LQ4_F16) return fail(LQ4_E_INVALID, "x_dtype must be LQ4_F32 or LQ4_F16");
    const uint8_t* wp;
    const int rc = resolve_weight_q8(w, w_extra_offset, n, k, &wp);
    if (rc) return rc;
    if (!x_dev || !y_dev) return fail(LQ4_E_INVALID, "x/y device pointer is null");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (m == 1 && x_dtype == LQ4_F32 && gemv_q8_lds_bytes(k) <= 128 * 1024) {
        launch_gemv_q8_b1(wp, n, k, static_cast<const float*>(x_dev), y_dev, s);
        ctx->counters.gemv++;
    } else if (m <= 32 || gemm_skinny_wants(n, k, m)) {
        // few rows: operands packed once, the few-token matrix-core kernel with this format's decoder
        // (always up to 32 rows: the large-tile kernels are no match for it there)
        const int src = ensure_scratch(ctx, gemm_skinny_scratch_bytes(k, m), static_cast<hipStream_t>(stream));
        if (src) return src;
        const LoraEpilogue none{nullptr, nullptr, 0, 0, 0.0f};
        launch_gemm_skinny(wp, n, k, x_dev, x_dtype == LQ4_F16, m, y_dev, none, ctx->moe_scratch, s, 1);
        ctx->counters.gemm++;
    } else {
        const int src = ensure_scratch(ctx, gemm_sibling_scratch_floats(1, n, k, m, ctx->gemm_kernel) * sizeof(float), static_cast<hipStream_t>(stream));
        if (src) return src;
        launch_gemm_q8(wp, n, k, x_dev, x_dtype == LQ4_F16, m, y_dev, reinterpret_cast<float*>(ctx->moe_scratch), ctx->gemm_kernel, s);
        ctx->counters.gemm++;
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_gemv_q8(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const float* x_dev, uint32_t batch, float* y_dev, void* stream) {
    if (batch > kMaxGemvBatch)
        return fail(LQ4_E_INVALID, "lq4_gemv_q8 batch %u above %d; use lq4_gemm_q8", batch, kMaxGemvBatch);
    return lq4_gemm_q8(ctx, w, w_extra_offset, n, k, x_dev, LQ4_F32, batch, y_dev, stream);
}

int lq4_gemm_q3(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const void* x_dev, int x_dtype, uint32_t m, float* y_dev, void* stream) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (m == 0 || n == 0) return LQ4_OK;
    if (x_dtype != LQ4_F32 && x_dtype != LQ4_F16) return fail(LQ4_E_INVALID, "x_dtype must be LQ4_F32 or LQ4_F16");
    const uint8_t* wp;
    const int rc = resolve_weight_sibling(w, w_extra_offset, n, k, "Q3", 16, 4, &wp);
    if (rc) return rc;
    if (!x_dev || !y_dev) return fail(LQ4_E_INVALID, "x/y device pointer is null");
    if (reinterpret_cast<uintptr_t>(x_dev) % 16) return fail(LQ4_E_INVALID, "x must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(y_dev) % 4) return fail(LQ4_E_INVALID, "y must be 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    DeviceGuard g(ctx->device);
    if (m == 1 && x_dtype == LQ4_F32 && gemv_q3_lds_bytes(k) <= 128 * 1024) {
        launch_gemv_q3_b1(wp, n, k, static_cast<const float*>(x_dev), y_dev, s);
        ctx->counters.gemv++;
    } else if (m <= 32 || gemm_skinny_wants(n, k, m)) {
        // few rows: operands packed once, the few-token matrix-core kernel with this format's decoder
        // (always up to 32 rows: the large-tile kernels are no match for it there)
        const int src = ensure_scratch(ctx, gemm_skinny_scratch_bytes(k, m), static_cast<hipStream_t>(stream));
        if (src) return src;
        const LoraEpilogue none{nullptr, nullptr, 0, 0, 0.0f};
        launch_gemm_skinny(wp, n, k, x_dev, x_dtype == LQ4_F16, m, y_dev, none, ctx->moe_scratch, s, 2);
        ctx->counters.gemm++;
    } else {
        const int src = ensure_scratch(ctx, gemm_sibling_scratch_floats(2, n, k, m, ctx->gemm_kernel) * sizeof(float), static_cast<hipStream_t>(stream));
        if (src) return src;
        launch_gemm_q3(wp, n, k, x_dev, x_dtype == LQ4_F16, m, y_dev, reinterpret_cast<float*>(ctx->moe_scratch), ctx->gemm_kernel, s);
        ctx->counters.gemm++;
    }
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_gemv_q3(lq4_ctx* ctx, const lq4_weight* w, uint64_t w_extra_offset, uint32_t n, uint32_t k,
                const float* x_dev, uint32_t batch, float* y_dev, void* stream) {
    if (batch > kMaxGemvBatch)
        return fail(LQ4_E_INVALID, "lq4_gemv_q3 batch %u above %d; use lq4_gemm_q3", batch, kMaxGemvBatch);
    return lq4_gemm_q3(ctx, w, w_extra_offset, n, k, x_dev, LQ4_F32, batch, y_dev, stream);
}

int lq4_set_gemv_kernel(lq4_ctx* ctx, int which) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (which < LQ4_GEMV_KERNEL_AUTO || which > LQ4_GEMV_KERNEL_LDS_RING)
        return fail(LQ4_E_INVALID, "gemv kernel choice must be 0..2");
    ctx->gemv_kernel = which;
    return LQ4_OK;
}

int lq4_set_gemm_kernel(lq4_ctx* ctx, int which) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    if (which < 0 || which > 4) return fail(LQ4_E_INVALID, "gemm kernel choice must be 0..4");
    ctx->gemm_kernel = which;
    return LQ4_OK;
}

int lq4_probe_copy(lq4_ctx* ctx, const void* src_dev, void* dst_dev, size_t nbytes, void* stream) {
    if (!ctx || !src_dev || !dst_dev) return fail(LQ4_E_INVALID, "null argument");
    if (reinterpret_cast<uintptr_t>(src_dev) % 16 || reinterpret_cast<uintptr_t>(dst_dev) % 16 || nbytes % 16)
        return fail(LQ4_E_INVALID, "buffers and size must be multiples of 16 bytes");
    DeviceGuard g(ctx->device);
    launch_probe_copy(src_dev, dst_dev, nbytes, static_cast<hipStream_t>(stream));
    LQ4_HIP(hipGetLastError());
    return LQ4_OK;
}

int lq4_get_path_counters(const lq4_ctx* ctx, lq4_path_counters* out) {
    if (!ctx || !out) return fail(LQ4_E_INVALID, "null argument");
    *out = ctx->counters;
    uint32_t fallbacks = 0;
    DeviceGuard g(ctx->device);
    LQ4_HIP(hipMemcpy(&fallbacks, ctx->lora_sync + 2, sizeof fallbacks, hipMemcpyDeviceToHost));
    out->lora_t_fallback = fallbacks;
    return LQ4_OK;
}

int lq4_malloc(lq4_ctx* ctx, size_t nbytes, void** out_dev) {
    if (!ctx || !out_dev) return fail(LQ4_E_INVALID, "null argument");
    DeviceGuard g(ctx->device);
    LQ4_HIP(hipMalloc(out_dev, nbytes ? nbytes : 4));
    return LQ4_OK;
}

int lq4_free(lq4_ctx* ctx, void* p_dev) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    DeviceGuard g(ctx->device);
    LQ4_HIP(hipFree(p_dev));
    return LQ4_OK;
}

int lq4_memcpy_h2d(lq4_ctx* ctx, void* dst_dev, const void* src_host, size_t nbytes) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    DeviceGuard g(ctx->device);
    LQ4_HIP(hipMemcpy(dst_dev, src_host, nbytes, hipMemcpyHostToDevice));
    return LQ4_OK;
}

int lq4_memcpy_d2h(lq4_ctx* ctx, void* dst_host, const void* src_dev, size_t nbytes) {
    if (!ctx) return fail(LQ4_E_INVALID, "ctx is null");
    DeviceGuard g(ctx->device);
    LQ4_HIP(hipMemcpy(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost));
    return LQ4_OK;
}

}  // extern "C"
