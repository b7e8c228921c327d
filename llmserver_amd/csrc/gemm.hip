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

// What the kernel does to its activations before the product (fused so that few-row steps need
// fewer launches):
//   PLAIN   X is bfloat16 [M, K].
//   NORM    X = rmsnorm(resid + delta) * norm_weight, not yet computed: the kernel forms
//           s = round(resid + delta) (32-bit sum, the new residual stream, written to resid_out by
//           the first workgroup), multiplies round(s * norm_weight) into the product and scales the
//           result by rsqrt(mean(s^2) + eps), which it gets from the same pass over s.
//   SWIGLU  X = silu(gate) * up with gate_up [M, 2K] (gate first), computed in 32-bit.
enum { PLAIN = 0, NORM = 1, SWIGLU = 2 };

struct Prologue {
    const bf16_t* second;        // NORM: delta (may be null); SWIGLU: unused (up follows gate in the row)
    const float* norm_weight;    // NORM: [K]
    bf16_t* resid_out;           // NORM: [M, K], written if second != null
    float eps;
};

// GATED: W stacks a gate matrix on an up matrix ([2I, K], gate first) and the result wanted is
// silu(x . gate^T) * (x . up^T), [M, I].  A workgroup then takes 8 gate rows and the 8 up rows that
// belong to them as its 16 rows of W, so both halves of a product meet in its epilogue and the
// activation costs no launch and no trip of the [M, 2I] intermediate through memory.
// CHUNK is the number of 32-wide k steps whose loads are issued together (0: 8 for the plain product
// of up to 32 rows, else 4); the launcher picks the one that divides a wavefront's share of K with
// the least waste.
template <int MT, typename OutT, int PRO, bool GATED = false, int CHUNK = 0>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                      OutT* __restrict__ y, int M, int N, int K, Prologue pro) {
    constexpr int CH = CHUNK ? CHUNK : (PRO != PLAIN || MT > 2) ? 4 : 8;
    __shared__ float partial[GEMM_WAVES][MT][256];
    __shared__ float squares[GEMM_WAVES][MT][16];
    extern __shared__ float norm_weight_lds[];                     // NORM: the norm weights, [K]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int n0 = blockIdx.x * (GATED ? 8 : 16);
    const int k_per_wave = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32 * 32;
    const int k_begin = min(K, wave * k_per_wave), k_end = min(K, k_begin + k_per_wave);
    const int x_stride = PRO == SWIGLU ? 2 * K : K;
    const int w_row = GATED ? (col < 8 ? min(n0 + col, N / 2 - 1) : N / 2 + min(n0 + col - 8, N / 2 - 1)) : min(n0 + col, N - 1);
    const bf16_t* wp = w + (size_t)w_row * K + 8 * quad;
    const bf16_t* xp[MT];
    const bf16_t* x2p[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const size_t row = (size_t)min(16 * t + col, M - 1);
        xp[t] = x + row * x_stride + 8 * quad;
        x2p[t] = PRO == SWIGLU ? xp[t] + K : (PRO == NORM && pro.second ? pro.second + row * K + 8 * quad : xp[t]);
    }
    if (PRO == NORM) {
        for (int i = threadIdx.x * 4; i < K; i += GEMM_WAVES * 64 * 4)
            *reinterpret_cast<f32x4*>(norm_weight_lds + i) = *reinterpret_cast<const f32x4*>(pro.norm_weight + i);
        __syncthreads();
    }
    f32x4 acc[MT];
    float sumsq[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
        sumsq[t] = 0.f;
    }

    // A chunk: the operands of CH consecutive k steps.  Chunks are loaded one ahead of the chunk
    // being multiplied, X first (it comes from cache) so that it never queues behind the weights.
    struct Chunk {
        bf16x8 a[CH];
        bf16x8 b[CH][MT];
        bf16x8 b2[PRO == PLAIN ? 1 : CH][PRO == PLAIN ? 1 : MT];
    };
    const int k_safe = K - 8;                      // a lane past the end reads the row's last 8 values and is zeroed
    const bool has_second = PRO == SWIGLU || (PRO == NORM && pro.second != nullptr);
    auto load_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int k = min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                c.b[u][t] = *reinterpret_cast<const bf16x8*>(xp[t] + k);
                if (PRO != PLAIN) c.b2[u][t] = *reinterpret_cast<const bf16x8*>(x2p[t] + k);
            }
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
            const int k = k0 + 32 * u + 8 * quad;
            const bool inside = k < k_end;
            bf16x8 a = c.a[u];
            if (!inside) a = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                bf16x8 b = c.b[u][t];
                if (PRO == SWIGLU) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float gate = (float)b[e];
                        b[e] = (bf16_t)(gate / (1.f + expf(-gate)) * (float)c.b2[u][t][e]);
                    }
                } else if (PRO == NORM) {
                    const int ks = min(k, k_safe);
                    const f32x4 w0 = *reinterpret_cast<const f32x4*>(norm_weight_lds + ks);
                    const f32x4 w1 = *reinterpret_cast<const f32x4*>(norm_weight_lds + ks + 4);
                    bf16x8 sum = b;
                    if (has_second) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) sum[e] = (bf16_t)((float)b[e] + (float)c.b2[u][t][e]);
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float v = inside ? (float)sum[e] : 0.f;
                        sumsq[t] += v * v;
                        b[e] = (bf16_t)(v * (e < 4 ? w0[e] : w1[e - 4]));
                    }
                    const int m = 16 * t + col;
                    if (has_second && blockIdx.x == 0 && inside && m < M)
                        *reinterpret_cast<bf16x8*>(pro.resid_out + (size_t)m * K + k) = sum;
                }
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t], 0, 0, 0);
            }
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
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][(4 * quad + r) + 16 * col] = acc[t][r];     // [m in tile][n in tile]
        if (PRO == NORM) {
            float sq = sumsq[t];
            sq += __shfl_xor(sq, 16, 64);
            sq += __shfl_xor(sq, 32, 64);
            if (quad == 0) squares[wave][t][col] = sq;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < MT * 256; e += GEMM_WAVES * 64) {
        const int t = e >> 8, in_tile = e & 255;
        const int m = 16 * t + (in_tile >> 4), n = n0 + (in_tile & 15);
        float total = 0.f;
#pragma unroll
        for (int v = 0; v < GEMM_WAVES; ++v) total += partial[v][t][in_tile];
        if (PRO == NORM) {
            float sq = 0.f;
#pragma unroll
            for (int v = 0; v < GEMM_WAVES; ++v) sq += squares[v][t][in_tile >> 4];
            total *= rsqrtf(sq / (float)K + pro.eps);
        }
        if (GATED) {
            const int j = in_tile & 15;
            if (j < 8) {
                float up = 0.f;
#pragma unroll
                for (int v = 0; v < GEMM_WAVES; ++v) up += partial[v][t][in_tile + 8];
                if (PRO == NORM) {
                    float sq = 0.f;
#pragma unroll
                    for (int v = 0; v < GEMM_WAVES; ++v) sq += squares[v][t][in_tile >> 4];
                    up *= rsqrtf(sq / (float)K + pro.eps);
                }
                if (m < M && n0 + j < N / 2) y[(size_t)m * (N / 2) + n0 + j] = (OutT)(total / (1.f + expf(-total)) * up);
            }
            continue;
        }
        if (m < M && n < N) y[(size_t)m * N + n] = (OutT)total;
    }
}

// Two tiles of W per wavefront (32 rows of W per workgroup, or 16 gate rows and their 16 up rows):
// every slice of X that a wavefront loads then meets twice as much of W, which matters because X,
// though it comes from cache, competes with the weight stream for the path into the compute unit
// (at 8 rows of X and one tile, X is a third of what a workgroup loads).  For M <= 16 only, and worth
// it only where N gives enough workgroups of this size to fill the chip.
// CH is the number of 32-wide k steps whose loads are issued together; the launcher picks the one
// that divides a wavefront's share of K with the least waste.
template <typename OutT, bool GATED, int CH>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_skinny_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                           OutT* __restrict__ y, int M, int N, int K) {
    __shared__ float partial[GEMM_WAVES][2][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int half = N / 2;                                        // GATED: rows of the gate matrix
    const int n0 = blockIdx.x * (GATED ? 16 : 32);
    const int k_per_wave = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32 * 32;
    const int k_begin = min(K, wave * k_per_wave), k_end = min(K, k_begin + k_per_wave);
    const int row0 = GATED ? min(n0 + col, half - 1) : min(n0 + col, N - 1);
    const int row1 = GATED ? half + min(n0 + col, half - 1) : min(n0 + 16 + col, N - 1);
    const bf16_t* wp0 = w + (size_t)row0 * K + 8 * quad;
    const bf16_t* wp1 = w + (size_t)row1 * K + 8 * quad;
    const bf16_t* xp = x + (size_t)min(col, M - 1) * K + 8 * quad;
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    struct Chunk {
        bf16x8 a0[CH], a1[CH], b[CH];
    };
    const int k_safe = K - 8;
    auto load_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < CH; ++u) c.b[u] = *reinterpret_cast<const bf16x8*>(xp + min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad);
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const int k = min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad;
            c.a0[u] = *reinterpret_cast<const bf16x8*>(wp0 + k);
            c.a1[u] = *reinterpret_cast<const bf16x8*>(wp1 + k);
        }
    };
    auto multiply_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < CH; ++u) {
            const bool inside = k0 + 32 * u + 8 * quad < k_end;
            bf16x8 a0 = c.a0[u], a1 = c.a1[u];
            if (!inside) {
                a0 = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
                a1 = a0;
            }
            acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, c.b[u], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, c.b[u], acc1, 0, 0, 0);
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
    for (int r = 0; r < 4; ++r) {
        partial[wave][0][(4 * quad + r) + 16 * col] = acc0[r];      // [m][n in tile]
        partial[wave][1][(4 * quad + r) + 16 * col] = acc1[r];
    }
    __syncthreads();
    const int e = threadIdx.x, tile = e >> 8, in_tile = e & 255;
    const int m = in_tile >> 4, j = in_tile & 15;
    if (GATED) {
        if (tile) return;
        float gate = 0.f, up = 0.f;
#pragma unroll
        for (int v = 0; v < GEMM_WAVES; ++v) {
            gate += partial[v][0][in_tile];
            up += partial[v][1][in_tile];
        }
        if (m < M && n0 + j < half) y[(size_t)m * half + n0 + j] = (OutT)(gate / (1.f + expf(-gate)) * up);
        return;
    }
    float total = 0.f;
#pragma unroll
    for (int v = 0; v < GEMM_WAVES; ++v) total += partial[v][tile][in_tile];
    const int n = n0 + 16 * tile + j;
    if (m < M && n < N) y[(size_t)m * N + n] = (OutT)total;
}

// The chunk size in 4..8 that wastes the fewest loads past the end of a wavefront's share of K.
static int best_chunk(int K) {
    const int steps = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32;          // k steps of one wavefront
    int chunk = 8, least = 1 << 30;
    for (int c = 8; c >= 4; --c) {
        const int waste = (steps + c - 1) / c * c - steps;
        if (waste < least) {
            least = waste;
            chunk = c;
        }
    }
    return chunk;
}

template <typename OutT, bool GATED>
static int launch_wide(const bf16_t* x, const bf16_t* w, OutT* y, int M, int N, int K, int workgroups, hipStream_t stream) {
    const int chunk = best_chunk(K);
    const dim3 grid(workgroups), block(GEMM_WAVES * 64);
    switch (chunk) {
        case 4: gemm_skinny_wide_kernel<OutT, GATED, 4><<<grid, block, 0, stream>>>(x, w, y, M, N, K); break;
        case 5: gemm_skinny_wide_kernel<OutT, GATED, 5><<<grid, block, 0, stream>>>(x, w, y, M, N, K); break;
        case 6: gemm_skinny_wide_kernel<OutT, GATED, 6><<<grid, block, 0, stream>>>(x, w, y, M, N, K); break;
        case 7: gemm_skinny_wide_kernel<OutT, GATED, 7><<<grid, block, 0, stream>>>(x, w, y, M, N, K); break;
        default: gemm_skinny_wide_kernel<OutT, GATED, 8><<<grid, block, 0, stream>>>(x, w, y, M, N, K); break;
    }
    LSA_LAUNCH_CHECK();
}

// Whether workgroups of two tiles suit `tiles` 16-row tiles of W: they halve the activations' share
// of the traffic, which saves `gain_percent` of the time (measured: about 15 with the gated epilogue,
// where one tile means two half tiles; for the plain product about 10 at 9 to 16 rows, 3 at 4 to 8
// and a loss below that), but must still fill the compute units in whole rounds.
static bool two_tiles_pay(int M, long tiles, int tiling, int gain_percent) {
    if (M > 16 || tiling == 1) return false;
    if (tiling == 2) return true;
    if (gain_percent <= 0) return false;
    static int units = 0;
    if (!units) {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) return false;
        units = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    const long rounds_one = (tiles + units - 1) / units, rounds_two = ((tiles + 1) / 2 + units - 1) / units;
    return 2 * rounds_two * (100 - gain_percent) < rounds_one * 100;
}

template <typename OutT, int PRO>
static int launch(const void* x, const void* w, void* y, int M, int N, int K, Prologue pro, int tiling, hipStream_t stream) {
    const dim3 grid((N + 15) / 16), block(GEMM_WAVES * 64);
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    if (PRO == PLAIN && two_tiles_pay(M, grid.x, tiling, M > 8 ? 10 : M >= 4 ? 3 : 0)) return launch_wide<OutT, false>(xb, wb, (OutT*)y, M, N, K, (N + 31) / 32, stream);
    const size_t lds = PRO == NORM ? (size_t)K * sizeof(float) : 0;
    if (M <= 16 && PRO == PLAIN) {
        switch (best_chunk(K)) {
            case 4: gemm_skinny_kernel<1, OutT, PLAIN, false, 4><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro); break;
            case 5: gemm_skinny_kernel<1, OutT, PLAIN, false, 5><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro); break;
            case 6: gemm_skinny_kernel<1, OutT, PLAIN, false, 6><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro); break;
            case 7: gemm_skinny_kernel<1, OutT, PLAIN, false, 7><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro); break;
            default: gemm_skinny_kernel<1, OutT, PLAIN, false, 8><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro); break;
        }
    } else if (M <= 16) gemm_skinny_kernel<1, OutT, PRO><<<grid, block, lds, stream>>>(xb, wb, (OutT*)y, M, N, K, pro);
    else if (PRO != PLAIN) return -1;
    else if (M <= 32) gemm_skinny_kernel<2, OutT, PLAIN><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro);
    else gemm_skinny_kernel<4, OutT, PLAIN><<<grid, block, 0, stream>>>(xb, wb, (OutT*)y, M, N, K, pro);
    LSA_LAUNCH_CHECK();
}

// out_float32: 0 writes bfloat16, 1 writes float32.  tiling: tiles of W per workgroup, 1 or 2 (2 only for
// M <= 16), or 0 to let the size decide.  Refuses (returns -1) what it cannot take.
LSA_EXPORT int lsa_gemm_skinny(int out_float32, const void* x, const void* w, void* y, int M, int N, int K, int tiling,
                               hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 != 0 || K < 8 || tiling < 0 || tiling > 2 || (tiling == 2 && M > 16)) return -1;
    Prologue pro = {nullptr, nullptr, nullptr, 0.f};
    return out_float32 ? launch<float, PLAIN>(x, w, y, M, N, K, pro, tiling, stream)
                       : launch<bf16_t, PLAIN>(x, w, y, M, N, K, pro, tiling, stream);
}

// Y = (silu(gate) * up) . W^T with gate_up [M, 2K]; M <= 16.
LSA_EXPORT int lsa_gemm_skinny_swiglu(const void* gate_up, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K % 8 != 0 || K < 8) return -1;
    Prologue pro = {nullptr, nullptr, nullptr, 0.f};
    return launch<bf16_t, SWIGLU>(gate_up, w, y, M, N, K, pro, 1, stream);
}

// Y = rmsnorm(resid + delta) * norm_weight . W^T; resid_out = resid + delta (delta may be null: then
// nothing is written and resid_out is ignored).  resid_out must not alias resid.  M <= 16, K <= 16384.
LSA_EXPORT int lsa_gemm_skinny_norm(int out_float32, const void* resid, const void* delta, const float* norm_weight, float eps,
                                    void* resid_out, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K % 8 != 0 || K < 8 || K > 16384 || (delta && resid_out == resid)) return -1;
    Prologue pro = {(const bf16_t*)delta, norm_weight, (bf16_t*)resid_out, eps};
    return out_float32 ? launch<float, NORM>(resid, w, y, M, N, K, pro, 1, stream) : launch<bf16_t, NORM>(resid, w, y, M, N, K, pro, 1, stream);
}

// hidden[M, I] = silu(x . gate^T) * (x . up^T) with gate_up [2I, K] (gate rows first); M <= 16, I a multiple of 8.
LSA_EXPORT int lsa_gemm_skinny_gated(const void* x, const void* gate_up, void* hidden, int M, int I, int K, int tiling,
                                     hipStream_t stream) {
    if (M <= 0 || I <= 0) return 0;
    if (M > 16 || K % 8 != 0 || K < 8 || I % 8 != 0 || tiling < 0 || tiling > 2) return -1;
    Prologue pro = {nullptr, nullptr, nullptr, 0.f};
    if (two_tiles_pay(M, I / 8, tiling, 15))
        return launch_wide<bf16_t, true>((const bf16_t*)x, (const bf16_t*)gate_up, (bf16_t*)hidden, M, 2 * I, K, (I + 15) / 16, stream);
    gemm_skinny_kernel<1, bf16_t, PLAIN, true><<<dim3(I / 8), dim3(GEMM_WAVES * 64), 0, stream>>>(
        (const bf16_t*)x, (const bf16_t*)gate_up, (bf16_t*)hidden, M, 2 * I, K, pro);
    LSA_LAUNCH_CHECK();
}
