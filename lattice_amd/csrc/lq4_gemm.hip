// Prefill GEMM over native Q4 blocks: Y[M,N] = X[M,K] . W[N,K]^T, f16 operands into
// MFMA, f32 accumulate.  Each k-step consumes exactly one Q4 block per weight row;
// the block is dequantised to f16 in registers ("half(f32(q)*d + b)", the rounding
// point of the reference's tiled kernel, shaders/gemm_q4_tiled.metal:57-66) and
// staged in LDS next to the f16 activation tile.
#include "lq4_internal.hpp"

namespace lq4 {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int BM = 128;  // activation rows (tokens) per workgroup
constexpr int BN = 128;  // weight rows (output features) per workgroup
constexpr int BK = 32;   // one Q4 block along K
constexpr int LDS_STRIDE = BK + 8;  // halfs; 80-byte rows keep ds_read_b128 conflict-free

__device__ __forceinline__ float load_b(const void* b, int is_f16, size_t idx) {
    return is_f16 ? static_cast<float>(static_cast<const _Float16*>(b)[idx])
                  : static_cast<const float*>(b)[idx];
}

template <bool X_F16>
__global__ __launch_bounds__(256) void gemm_q4_mfma(const uint8_t* __restrict__ w, uint32_t n,
                                                    uint32_t k, const void* __restrict__ xv,
                                                    uint32_t m, float* __restrict__ y,
                                                    LoraEpilogue lora) {
    __shared__ __attribute__((aligned(16))) _Float16 Xs[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) _Float16 Ws[BN * LDS_STRIDE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = (wave >> 1) * 64;  // wave's 64x64 sub-tile inside the 128x128 tile
    const int wn = (wave & 1) * 64;
    const uint32_t m0 = blockIdx.y * BM;
    const uint32_t n0 = blockIdx.x * BN;
    const uint32_t nb = k / kBlockWeights;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;

    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- global -> register staging -------------------------------------------------
    // activations: f16 -> 2 x 16-byte chunks per thread; f32 -> 4 x 16-byte chunks
    constexpr int XCH = X_F16 ? 2 : 4;
    uint4 xreg[XCH];
    uint32_t wreg[5];
    const bool w_loader = tid < BN;
    const uint32_t w_row = n0 + tid;
    const uint8_t* w_ptr = w + static_cast<size_t>(w_row < n ? w_row : 0) * row_bytes;

    auto load_tiles = [&](uint32_t kb) {
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            const int c = tid + 256 * i;
            if (X_F16) {
                const int row = c >> 2, part = c & 3;
                const uint32_t gm = m0 + row;
                xreg[i] = gm < m ? *reinterpret_cast<const uint4*>(static_cast<const _Float16*>(xv) +
                                                                   static_cast<size_t>(gm) * k + kb * BK + part * 8)
                                 : make_uint4(0, 0, 0, 0);
            } else {
                const int row = c >> 3, part = c & 7;
                const uint32_t gm = m0 + row;
                xreg[i] = gm < m ? *reinterpret_cast<const uint4*>(static_cast<const float*>(xv) +
                                                                   static_cast<size_t>(gm) * k + kb * BK + part * 4)
                                 : make_uint4(0, 0, 0, 0);
            }
        }
        if (w_loader) {
            const uint32_t* p = reinterpret_cast<const uint32_t*>(w_ptr + static_cast<size_t>(kb) * kBlockBytes);
#pragma unroll
            for (int i = 0; i < 5; ++i) wreg[i] = p[i];
        }
    };

    auto store_tiles = [&]() {
#pragma unroll
        for (int i = 0; i < XCH; ++i) {
            const int c = tid + 256 * i;
            if (X_F16) {
                const int row = c >> 2, part = c & 3;
                *reinterpret_cast<uint4*>(&Xs[row * LDS_STRIDE + part * 8]) = xreg[i];
            } else {
                const int row = c >> 3, part = c & 7;
                half4 h;
                h[0] = static_cast<_Float16>(__builtin_bit_cast(float, xreg[i].x));
                h[1] = static_cast<_Float16>(__builtin_bit_cast(float, xreg[i].y));
                h[2] = static_cast<_Float16>(__builtin_bit_cast(float, xreg[i].z));
                h[3] = static_cast<_Float16>(__builtin_bit_cast(float, xreg[i].w));
                *reinterpret_cast<half4*>(&Xs[row * LDS_STRIDE + part * 4]) = h;
            }
        }
        if (w_loader) {
            const bool live = w_row < n;
            const float d = live ? f16_bits_to_f32(wreg[0] & 0xffffu) : 0.0f;
            const float b = live ? f16_bits_to_f32(wreg[0] >> 16) : 0.0f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t q = wreg[1 + j];
                half8 h;
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    h[i] = static_cast<_Float16>(fmaf(static_cast<float>((q >> (4 * i)) & 0xfu), d, b));
                *reinterpret_cast<half8*>(&Ws[tid * LDS_STRIDE + j * 8]) = h;
            }
        }
    };

    load_tiles(0);
    for (uint32_t kb = 0; kb < nb; ++kb) {
        store_tiles();
        __syncthreads();
        if (kb + 1 < nb) load_tiles(kb + 1);
        // operand layout of v_mfma_f32_32x32x16_f16: lane l supplies row/col (l & 31),
        // k-slice 8*(l >> 5) .. +7 of a 16-deep step
        const int r = lane & 31, ks = (lane >> 5) * 8;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            half8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i] = *reinterpret_cast<const half8*>(&Xs[(wm + i * 32 + r) * LDS_STRIDE + kk + ks]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j] = *reinterpret_cast<const half8*>(&Ws[(wn + j * 32 + r) * LDS_STRIDE + kk + ks]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // ---- epilogue: accumulator element v of lane l is
    //      row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t gn = n0 + wn + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t gm = m0 + wm + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (gm < m && gn < n) {
                    float val = acc[i][j][v];
                    if (lora.rank) {
                        float s = 0.0f;
                        for (uint32_t jj = 0; jj < lora.rank; ++jj)
                            s += load_b(lora.b, lora.b_is_f16, static_cast<size_t>(gn) * lora.rank + jj) *
                                 lora.t[static_cast<size_t>(gm) * lora.rank + jj];
                        val += lora.scale * s;
                    }
                    y[static_cast<size_t>(gm) * n + gn] = val;
                }
            }
        }
}

}  // namespace

void launch_gemm(const uint8_t* w, uint32_t n, uint32_t k, const void* x, int x_is_f16, uint32_t m,
                 float* y, const LoraEpilogue& lora, hipStream_t stream) {
    const dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM), block(256);
    if (x_is_f16)
        hipLaunchKernelGGL(gemm_q4_mfma<true>, grid, block, 0, stream, w, n, k, x, m, y, lora);
    else
        hipLaunchKernelGGL(gemm_q4_mfma<false>, grid, block, 0, stream, w, n, k, x, m, y, lora);
}

}  // namespace lq4
