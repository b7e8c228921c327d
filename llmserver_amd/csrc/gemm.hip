// Weight-streaming matrix product for a few rows of activations (decode steps):
//   Y[M, N] = X[M, K] . W[N, K]^T,  bfloat16 inputs, 32-bit accumulation, M <= 64.
// With so few rows the product is bound by reading W once from HBM, so the kernel is built
// around that stream: a workgroup owns 16 consecutive rows of W (16 output columns); its eight
// wavefronts split K between them, each streams its slice of the 16 rows with 16-byte loads
// issued many at a time, multiplies it with the matching slice of X (which stays in cache) on
// 16x16x32 MFMAs, and the eight partial tiles are added through LDS and rounded once.
//   MFMA operands (lane = 16 * quad + col):  A = W rows   (lane: row n0 + col, 8 k of quad)
//                                            B = X^T      (lane: row 16 t + col of X, same k)
//   result lane holds Y^T[n0 + 4 quad + r][16 t + col].
#include "common.hpp"

using namespace lsa;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int GEMM_WAVES = 8;

template <int MT, typename OutT>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                      OutT* __restrict__ y, int M, int N, int K) {
    constexpr int CH = MT <= 2 ? 8 : 4;          // 32-wide k steps loaded together (one chunk)
    __shared__ float partial[GEMM_WAVES][MT][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int k_per_wave = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32 * 32;
    const int k_begin = min(K, wave * k_per_wave), k_end = min(K, k_begin + k_per_wave);
    const bf16_t* wp = w + (size_t)min(n0 + col, N - 1) * K + 8 * quad;
    const bf16_t* xp[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xp[t] = x + (size_t)min(16 * t + col, M - 1) * K + 8 * quad;
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // A chunk: the operands of CH consecutive k steps.  Chunks are loaded one ahead of the chunk
    // being multiplied, X first (it comes from cache) so that it never queues behind the weights.
    struct Chunk {
        bf16x8 a[CH];
        bf16x8 b[CH][MT];
    };
    const int k_safe = K - 8;                      // a lane past the end reads the row's last 8 values and is zeroed
    auto load_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int k = min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad;
#pragma unroll
            for (int t = 0; t < MT; ++t) c.b[u][t] = *reinterpret_cast<const bf16x8*>(xp[t] + k);
        }
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int k = min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad;
            c.a[u] = *reinterpret_cast<const bf16x8*>(wp + k);
        }
    };
    auto multiply_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            bf16x8 a = c.a[u];
            if (k0 + 32 * u + 8 * quad >= k_end) a = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, c.b[u][t], acc[t], 0, 0, 0);
        }
    };
    if (k_begin < k_end) {
        constexpr int SPAN = 32 * CH;
        Chunk p, q;
        int k0 = k_begin;
        int chunks = (k_end - k_begin + SPAN - 1) / SPAN;
        load_chunk(p, k0);
        while (chunks >= 3) {
            load_chunk(q, k0 + SPAN);
            multiply_chunk(p, k0);
            load_chunk(p, k0 + 2 * SPAN);
            multiply_chunk(q, k0 + SPAN);
            k0 += 2 * SPAN;
            chunks -= 2;
        }
        if (chunks == 2) {
            load_chunk(q, k0 + SPAN);
            multiply_chunk(p, k0);
            multiply_chunk(q, k0 + SPAN);
        } else {
            multiply_chunk(p, k0);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][(4 * quad + r) + 16 * col] = acc[t][r];     // [m in tile][n in tile]
    __syncthreads();
    for (int e = threadIdx.x; e < MT * 256; e += GEMM_WAVES * 64) {
        const int t = e >> 8, in_tile = e & 255;
        const int m = 16 * t + (in_tile >> 4), n = n0 + (in_tile & 15);
        float total = 0.f;
#pragma unroll
        for (int v = 0; v < GEMM_WAVES; ++v) total += partial[v][t][in_tile];
        if (m < M && n < N) y[(size_t)m * N + n] = (OutT)total;
    }
}

template <typename OutT>
static int launch(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
    const dim3 grid((N + 15) / 16), block(GEMM_WAVES * 64);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    if (M <= 16) gemm_skinny_kernel<1, OutT><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K);
    else if (M <= 32) gemm_skinny_kernel<2, OutT><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K);
    else gemm_skinny_kernel<4, OutT><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K);
    LSA_LAUNCH_CHECK();
}

// out_float32: 0 writes bfloat16, 1 writes float32.  Refuses (returns -1) what it cannot take.
LSA_EXPORT int lsa_gemm_skinny(int out_float32, const void* x, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 != 0 || K < 8) return -1;
    return out_float32 ? launch<float>(x, w, y, M, N, K, stream) : launch<bf16_t>(x, w, y, M, N, K, stream);
}
