/*
 * cpu_baseline.c — the reference's CPU route for a Q4 matmul, restated in C so it
 * can be timed on the GPU box's host cores next to the HIP kernels.
 *
 * TEST/BENCH INFRASTRUCTURE ONLY (bench.py's cpu_baseline leg and tests/); the
 * shipped library never links or calls it.
 *
 * The reference has no CPU Q4 kernel: a Q4 tensor reaches the CPU by
 * dequantize_row_q4_0 (crates/inference/src/weights/q4_weights.rs:340-353)
 * into f32 and then the f32 `matmul_bt` C = A.B^T
 * (crates/inference/src/forward/cpu/matmul.rs:59-121).  On non-macOS x86-64
 * that dispatcher is single-threaded and picks, in order:
 *   m*n*k >= 2^20 and k >= 128 -> cache-blocked 4x8x128 tiles, whose AVX2
 *       micro-kernel only runs on full 4x8 tiles; every other tile (so every
 *       tile when m < 4) takes the scalar edge loop (tiled.rs:17-58,
 *       tiled_avx2.rs:47, 258-272);
 *   else AVX-512F dot (arch_kernels.rs:80-140) if the CPU has it;
 *   else AVX2+FMA dot, 4 accumulators x 8 lanes (arch_kernels.rs:12-66);
 *   else scalar.
 * Build: gcc -O3 -mavx2 -mfma (+ -mavx512f for the one function that needs it,
 * selected at run time with __builtin_cpu_supports).
 */
#include <immintrin.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define TILE_I 4
#define TILE_J 8
#define TILE_K 128

size_t lq4o_dequantize(const uint8_t* data, size_t nbytes, size_t n_weights, float* out);

/* arch_kernels.rs:222-228 */
static inline float hsum8(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehdup_ps(s));
    return _mm_cvtss_f32(_mm_add_ss(s, _mm_movehl_ps(s, s)));
}

/* arch_kernels.rs:22-65 */
static float dot_avx2(const float* a, const float* b, size_t len) {
    __m256 acc[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(),
                     _mm256_setzero_ps()};
    size_t chunks = len / 32;
    for (size_t c = 0; c < chunks; ++c)
        for (int u = 0; u < 4; ++u)
            acc[u] = _mm256_fmadd_ps(_mm256_loadu_ps(a + c * 32 + u * 8),
                                     _mm256_loadu_ps(b + c * 32 + u * 8), acc[u]);
    float sum = hsum8(_mm256_add_ps(_mm256_add_ps(acc[0], acc[1]), _mm256_add_ps(acc[2], acc[3])));
    size_t off = chunks * 32, end8 = (len / 8) * 8;
    for (; off < end8; off += 8)
        sum += hsum8(_mm256_mul_ps(_mm256_loadu_ps(a + off), _mm256_loadu_ps(b + off)));
    for (; off < len; ++off) sum += a[off] * b[off];
    return sum;
}

/* arch_kernels.rs:12-21 */
void lq4o_matmul_bt_avx2(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) c[i * n + j] = dot_avx2(a + i * k, b + j * k, k);
}

/* arch_kernels.rs:80-140 */
__attribute__((target("avx512f"))) static float dot_avx512(const float* a, const float* b,
                                                            size_t len) {
    __m512 acc[4] = {_mm512_setzero_ps(), _mm512_setzero_ps(), _mm512_setzero_ps(),
                     _mm512_setzero_ps()};
    size_t chunks = len / 64;
    for (size_t c = 0; c < chunks; ++c)
        for (int u = 0; u < 4; ++u)
            acc[u] = _mm512_fmadd_ps(_mm512_loadu_ps(a + c * 64 + u * 16),
                                     _mm512_loadu_ps(b + c * 64 + u * 16), acc[u]);
    float sum = _mm512_reduce_add_ps(
        _mm512_add_ps(_mm512_add_ps(acc[0], acc[1]), _mm512_add_ps(acc[2], acc[3])));
    size_t off = chunks * 64, end16 = (len / 16) * 16;
    for (; off < end16; off += 16)
        sum += _mm512_reduce_add_ps(_mm512_mul_ps(_mm512_loadu_ps(a + off), _mm512_loadu_ps(b + off)));
    for (; off < len; ++off) sum += a[off] * b[off];
    return sum;
}

__attribute__((target("avx512f"))) void lq4o_matmul_bt_avx512(const float* a, const float* b,
                                                              float* c, size_t m, size_t k,
                                                              size_t n) {
    for (size_t i = 0; i < m; ++i)
        for (size_t j = 0; j < n; ++j) c[i * n + j] = dot_avx512(a + i * k, b + j * k, k);
}

/* tiled_avx2.rs:17-285 — j-tiles outermost, then i-tiles, then k-tiles of 128;
 * a full 4x8 tile with >= 16 k-values keeps 32 eight-lane accumulators and adds
 * their horizontal sums into C; anything else runs the scalar edge loop. */
void lq4o_matmul_bt_tiled_avx2(const float* a, const float* b, float* c, size_t m, size_t k,
                               size_t n) {
    memset(c, 0, m * n * sizeof(float));
    for (size_t j0 = 0; j0 < n; j0 += TILE_J) {
        size_t jc = n - j0 < TILE_J ? n - j0 : TILE_J;
        for (size_t i0 = 0; i0 < m; i0 += TILE_I) {
            size_t ic = m - i0 < TILE_I ? m - i0 : TILE_I;
            for (size_t k0 = 0; k0 < k; k0 += TILE_K) {
                size_t k1 = k0 + TILE_K < k ? k0 + TILE_K : k;
                size_t klen = k1 - k0;
                if (ic == TILE_I && jc == TILE_J && klen >= 16) {
                    __m256 acc[TILE_I][TILE_J];
                    for (int i = 0; i < TILE_I; ++i)
                        for (int j = 0; j < TILE_J; ++j) acc[i][j] = _mm256_setzero_ps();
                    size_t kvec = (klen / 8) * 8;
                    for (size_t kk = 0; kk < kvec; kk += 8) {
                        __m256 bv[TILE_J];
                        for (int j = 0; j < TILE_J; ++j)
                            bv[j] = _mm256_loadu_ps(b + (j0 + j) * k + k0 + kk);
                        for (int i = 0; i < TILE_I; ++i) {
                            __m256 av = _mm256_loadu_ps(a + (i0 + i) * k + k0 + kk);
                            for (int j = 0; j < TILE_J; ++j)
                                acc[i][j] = _mm256_fmadd_ps(av, bv[j], acc[i][j]);
                        }
                    }
                    for (int i = 0; i < TILE_I; ++i)
                        for (int j = 0; j < TILE_J; ++j)
                            c[(i0 + i) * n + j0 + j] += hsum8(acc[i][j]);
                    for (int i = 0; i < TILE_I && k0 + kvec < k1; ++i)
                        for (int j = 0; j < TILE_J; ++j) {
                            float s = 0.0f;
                            for (size_t p = k0 + kvec; p < k1; ++p)
                                s += a[(i0 + i) * k + p] * b[(j0 + j) * k + p];
                            c[(i0 + i) * n + j0 + j] += s;
                        }
                } else {
                    for (size_t i = 0; i < ic; ++i)
                        for (size_t j = 0; j < jc; ++j) {
                            float s = 0.0f;
                            for (size_t p = k0; p < k1; ++p)
                                s += a[(i0 + i) * k + p] * b[(j0 + j) * k + p];
                            c[(i0 + i) * n + j0 + j] += s;
                        }
                }
            }
        }
    }
}

/* matmul.rs:59-121, non-macOS x86-64 arm.  Returns which kernel ran:
 * 0 tiled (AVX2 micro-kernel / scalar edges), 1 AVX-512F dot, 2 AVX2 dot. */
int lq4o_matmul_bt(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    unsigned long long work = (unsigned long long)m * n * k;
    if (work >= 1024ull * 1024ull && k >= TILE_K) {
        lq4o_matmul_bt_tiled_avx2(a, b, c, m, k, n);
        return 0;
    }
    if (__builtin_cpu_supports("avx512f")) {
        lq4o_matmul_bt_avx512(a, b, c, m, k, n);
        return 1;
    }
    lq4o_matmul_bt_avx2(a, b, c, m, k, n);
    return 2;
}

/* The whole CPU route for one Q4 weight matrix: dequantize every row to f32
 * (w_f32 is caller scratch of n*k floats), then matmul_bt.  `mode` 0 = the
 * reference dispatch, 1 = force the AVX2 dot kernel.  Returns the kernel id. */
int lq4o_cpu_q4_matmul(const float* x, const uint8_t* wq, float* w_f32, float* y, size_t m,
                       size_t n, size_t k, int mode, int skip_dequant) {
    size_t row_bytes = (k / 32) * 20;
    if (!skip_dequant)
        for (size_t r = 0; r < n; ++r) lq4o_dequantize(wq + r * row_bytes, row_bytes, k, w_f32 + r * k);
    if (mode == 1) {
        lq4o_matmul_bt_avx2(x, w_f32, y, m, k, n);
        return 2;
    }
    return lq4o_matmul_bt(x, w_f32, y, m, k, n);
}
