// Weight-streaming matrix products for a few rows of activations (decode steps, short portions):
//   Y[M, N] = X[M, K] . W[N, K]^T,  bfloat16 inputs, 32-bit accumulation.
// With so few rows the product is bound by reading W once from HBM, so the kernels are built
// around that stream.  Two families: the one below for up to 16 rows (it runs up to 64, but is
// beaten there), and further down one for 17 to 128 rows that leaves partial sums.
// In the first, a workgroup owns 16 (or 32) consecutive rows of W; its eight wavefronts
// split K between them, each streams its slice of the rows with 16-byte loads issued many at a
// time, multiplies it with the matching slice of X (which stays in cache) on 16x16x32 MFMAs, and
// the eight partial tiles are added through LDS and rounded once.
//   MFMA operands (lane = 16 * quad + col):  A = W rows   (lane: row n0 + col, 8 k of quad)
//                                            B = X^T      (lane: row 16 t + col of X, same k)
//   result lane holds Y^T[n0 + 4 quad + r][16 t + col].
//
// Around the product, for up to 16 rows, two things can be fused that would otherwise be kernels
// of their own between two products (each costs a launch and a trip of the rows through memory):
//   * Row scale.  X = s * w for a residual stream s and a norm's weights w, and the result wanted
//     is rmsnorm(s) * w . W^T = (X . W^T) / rms(s).  The kernel is given partial sums of s^2
//     ([M, P], any split of a row into P parts) and multiplies its result rows by
//     rsqrt(sum / K + eps) in the epilogue.
//   * Stream update.  The result is an update of a residual stream that a norm follows.  The
//     epilogue then forms s' = round(resid + round(y)), and writes s', round(s' * norm_weight) and
//     the sum of s'^2 over the columns of each workgroup ([M, P]): exactly what the row scale of the
//     next product takes.
#include "common.hpp"

using namespace lsa;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int GEMM_WAVES = 8;
constexpr int FUSED_ROWS = 16;           // most rows the fused epilogues take (each of the 8 wavefronts finds the scale of two rows)
constexpr int SCALE_PARTS = 512;         // most partial sums per row the row scale takes (half as many from 9 rows on)

struct Fusion {
    // Row scale (null: none).
    const float* square_sums;            // [M, n_parts]
    int n_parts;
    float eps;
    // Stream update (resid null: none); bfloat16 results only.
    const bf16_t* resid;                 // [M, N]
    const float* norm_weight;            // [N]
    bf16_t* resid_out;                   // [M, N]
    bf16_t* weighted_out;                // [M, N]
    float* square_sums_out;              // [M, P], P as lsa_gemm_skinny_parts tells
    // Bias (null: none), added to the float32 sum before its one rounding; plain results only.
    const float* bias;                   // [N]
};

// The partial sums of wavefront `wave`'s row are loaded behind the last operands of the product
// (they come from cache and are there by the time those have arrived) and while few registers
// are in use; the loads are issued whether or not a scale was asked for, from a harmless address
// if not, so that no branch stands between the loads of the product and the waits for them.
// Wavefront `wave` finds the scale of row `wave` from up to 512 partial sums, or, from 9 rows on, the
// scales of rows `wave` and `wave + 8` from up to 256 each: eight loads per lane either way.
struct RowScaleLoads {
    float part[SCALE_PARTS / 64];
};
__device__ inline int row_scale_row(int M, int wave, int i) { return M <= GEMM_WAVES ? wave : wave + GEMM_WAVES * (i >> 2); }
__device__ inline int row_scale_part(int M, int lane, int i) { return M <= GEMM_WAVES ? lane + 64 * i : lane + 64 * (i & 3); }
__device__ inline void row_scale_issue(RowScaleLoads& loads, const Fusion& f, const void* harmless, int M, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < SCALE_PARTS / 64; ++i) {
        const int row = row_scale_row(M, wave, i);
        const bool wanted = f.square_sums && row < M;
        const float* src = wanted ? f.square_sums + (size_t)row * f.n_parts : (const float*)harmless;
        loads.part[i] = src[wanted ? min(row_scale_part(M, lane, i), f.n_parts - 1) : 0];
    }
}
// 1 / rms of the wavefront's row or rows into scale[row].
__device__ inline void row_scale_finish(const RowScaleLoads& loads, const Fusion& f, int M, int K, int wave, int lane, float* scale) {
    if (!f.square_sums) return;
    float sum[2] = {0.f, 0.f};
#pragma unroll
    for (int i = 0; i < SCALE_PARTS / 64; ++i)
        sum[M <= GEMM_WAVES ? 0 : i >> 2] += row_scale_part(M, lane, i) < f.n_parts ? loads.part[i] : 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = wave + GEMM_WAVES * h;
        if (row >= M || (h && M <= GEMM_WAVES)) continue;
        const float total = wave_sum(sum[h]);
        if (lane == 0) scale[row] = rsqrtf(total / (float)K + f.eps);
    }
}

// Epilogue of the stream update for one element (m, n) of the result; the 16 lanes that hold
// the 16 columns of a tile for one m are neighbours, so the sum of squares is four shuffles.
__device__ inline float stream_update(const Fusion& f, float total, int m, int n, int M, int N, bool own) {
    const bool inside = own && m < M && n < N;
    float s = 0.f;
    if (inside) {
        const size_t at = (size_t)m * N + n;
        const bf16_t updated = (bf16_t)((float)f.resid[at] + (float)(bf16_t)total);
        s = (float)updated;
        f.resid_out[at] = updated;
        f.weighted_out[at] = (bf16_t)(s * f.norm_weight[n]);
    }
    float sq = s * s;
    sq += __shfl_xor(sq, 1, 64);
    sq += __shfl_xor(sq, 2, 64);
    sq += __shfl_xor(sq, 4, 64);
    sq += __shfl_xor(sq, 8, 64);
    return sq;                              // the tile's sum for row m, in all 16 lanes that hold the row
}

// One tile of W per workgroup.  GATED: W stacks a gate matrix on an up matrix ([2I, K], gate first)
// and the result wanted is silu(x . gate^T) * (x . up^T), [M, I]; the workgroup then takes 8 gate
// rows and the 8 up rows that belong to them as its 16 rows of W, so both halves of a product meet
// in its epilogue.  CH is the number of 32-wide k steps whose loads are issued together; the
// launcher picks the one that divides a wavefront's share of K with the least waste.
template <int MT, typename OutT, bool GATED, int CH>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                      OutT* __restrict__ y, int M, int N, int K, int R, Fusion fusion) {
    __shared__ float partial[GEMM_WAVES][MT][256];
    __shared__ float row_scale[FUSED_ROWS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    // R of the tile's 16 rows are this workgroup's own (GATED: 8 gate rows and 8 up rows); the other lanes
    // load the last of them again, which costs no traffic, and their results are dropped.
    const int n0 = blockIdx.x * (GATED ? 8 : R);
    const int k_per_wave = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32 * 32;
    const int k_begin = min(K, wave * k_per_wave), k_end = min(K, k_begin + k_per_wave);
    const int w_row = GATED ? (col < 8 ? min(n0 + col, N / 2 - 1) : N / 2 + min(n0 + col - 8, N / 2 - 1))
                            : min(n0 + min(col, R - 1), N - 1);
    const bf16_t* wp = w + (size_t)w_row * K + 8 * quad;
    const bf16_t* xp[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xp[t] = x + (size_t)min(16 * t + col, M - 1) * K + 8 * quad;
    RowScaleLoads scale_loads;
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
        // The scheduling barriers keep a chunk's loads together and ahead of the products of the chunk before: left to
        // itself the compiler spreads them between those products, a few at a time, each group waited for (down to "no
        // load in flight") right behind the products it was issued between (output product of 4096 x 4096 at 8 rows
        // 9.9 -> 8.8 us, down product 25.0 -> 24.0 us; in the two-tile kernel below they gain nothing).
        while (chunks >= 3) {
            load_chunk(q, k0 + SPAN);
            __builtin_amdgcn_sched_barrier(0);
            multiply_chunk(p, k0);
            __builtin_amdgcn_sched_barrier(0);
            load_chunk(p, k0 + 2 * SPAN);
            __builtin_amdgcn_sched_barrier(0);
            multiply_chunk(q, k0 + SPAN);
            __builtin_amdgcn_sched_barrier(0);
            k0 += 2 * SPAN;
            chunks -= 2;
        }
        if (chunks == 2) {
            load_chunk(q, k0 + SPAN);
            multiply_chunk(p, k0);
            if (MT == 1) row_scale_issue(scale_loads, fusion, x, M, wave, lane);
            multiply_chunk(q, k0 + SPAN);
        } else {
            if (MT == 1) row_scale_issue(scale_loads, fusion, x, M, wave, lane);
            multiply_chunk(p, k0);
        }
    } else if (MT == 1) {
        row_scale_issue(scale_loads, fusion, x, M, wave, lane);
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[wave][t][(4 * quad + r) + 16 * col] = acc[t][r];     // [m in tile][n in tile]
    if (MT == 1) row_scale_finish(scale_loads, fusion, M, K, wave, lane, row_scale);
    __syncthreads();
    for (int e = threadIdx.x; e < MT * 256; e += GEMM_WAVES * 64) {
        const int t = e >> 8, in_tile = e & 255;
        const int m = 16 * t + (in_tile >> 4), j = in_tile & 15, n = n0 + j;
        float total = 0.f;
#pragma unroll
        for (int v = 0; v < GEMM_WAVES; ++v) total += partial[v][t][in_tile];
        const float scale = (MT == 1 && fusion.square_sums && m < FUSED_ROWS) ? row_scale[m] : 1.f;
        total *= scale;
        if (GATED) {
            if (j < 8) {
                float up = 0.f;
#pragma unroll
                for (int v = 0; v < GEMM_WAVES; ++v) up += partial[v][t][in_tile + 8];
                up *= scale;
                if (m < M && n < N / 2) y[(size_t)m * (N / 2) + n] = (OutT)(total / (1.f + expf(-total)) * up);
            }
            continue;
        }
        if (MT == 1 && sizeof(OutT) == 2 && fusion.resid) {
            const float sq = stream_update(fusion, total, m, n, M, N, j < R);
            if (j == 0 && m < M) fusion.square_sums_out[(size_t)m * gridDim.x + blockIdx.x] = sq;
            continue;
        }
        if (m < M && j < R && n < N) y[(size_t)m * N + n] = (OutT)(fusion.bias ? total + fusion.bias[n] : total);
    }
}

// Two tiles of W per wavefront (32 rows of W per workgroup, or 16 gate rows and their 16 up rows):
// every slice of X that a wavefront loads then meets twice as much of W, which matters because X,
// though it comes from cache, competes with the weight stream for the path into the compute unit
// (at 8 rows of X and one tile, X is a third of what a workgroup loads).  For M <= 16 only, and worth
// it only where N gives enough workgroups of this size to fill the chip.
template <typename OutT, bool GATED, int CH>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_skinny_wide_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                           OutT* __restrict__ y, int M, int N, int K, int R, Fusion fusion) {
    __shared__ float partial[GEMM_WAVES][2][256];
    __shared__ float row_scale[FUSED_ROWS];
    __shared__ float second_tile_sums[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int half = N / 2;                                        // GATED: rows of the gate matrix
    // The workgroup's own rows: R (16 < R <= 32) consecutive ones, 16 in the first tile; GATED: R <= 16 gate rows
    // in the first tile, their up rows in the second.  Lanes beyond them load the last own row again.
    const int n0 = blockIdx.x * R;
    const int own0 = GATED ? R : 16, own1 = GATED ? R : R - 16;                     // own rows of the two tiles
    const int k_per_wave = ((K + GEMM_WAVES - 1) / GEMM_WAVES + 31) / 32 * 32;
    const int k_begin = min(K, wave * k_per_wave), k_end = min(K, k_begin + k_per_wave);
    const int row0 = GATED ? min(n0 + min(col, own0 - 1), half - 1) : min(n0 + col, N - 1);
    const int row1 = GATED ? half + min(n0 + min(col, own1 - 1), half - 1) : min(n0 + 16 + min(col, own1 - 1), N - 1);
    const bf16_t* wp0 = w + (size_t)row0 * K + 8 * quad;
    const bf16_t* wp1 = w + (size_t)row1 * K + 8 * quad;
    const bf16_t* xp = x + (size_t)min(col, M - 1) * K + 8 * quad;
    RowScaleLoads scale_loads;
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
            bf16x8 a0 = c.a0[u], a1 = c.a1[u];
            if (k0 + 32 * u + 8 * quad >= k_end) {
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
            row_scale_issue(scale_loads, fusion, x, M, wave, lane);
            multiply_chunk(q, k0 + SPAN);
        } else {
            row_scale_issue(scale_loads, fusion, x, M, wave, lane);
            multiply_chunk(p, k0);
        }
    } else {
        row_scale_issue(scale_loads, fusion, x, M, wave, lane);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        partial[wave][0][(4 * quad + r) + 16 * col] = acc0[r];      // [m][n in tile]
        partial[wave][1][(4 * quad + r) + 16 * col] = acc1[r];
    }
    row_scale_finish(scale_loads, fusion, M, K, wave, lane, row_scale);
    __syncthreads();
    const int e = threadIdx.x, tile = e >> 8, in_tile = e & 255;
    const int m = in_tile >> 4, j = in_tile & 15;
    const float scale = (fusion.square_sums && m < FUSED_ROWS) ? row_scale[m] : 1.f;
    if (GATED) {
        if (tile) return;
        float gate = 0.f, up = 0.f;
#pragma unroll
        for (int v = 0; v < GEMM_WAVES; ++v) {
            gate += partial[v][0][in_tile];
            up += partial[v][1][in_tile];
        }
        gate *= scale;
        up *= scale;
        if (m < M && j < own0 && n0 + j < half) y[(size_t)m * half + n0 + j] = (OutT)(gate / (1.f + expf(-gate)) * up);
        return;
    }
    float total = 0.f;
#pragma unroll
    for (int v = 0; v < GEMM_WAVES; ++v) total += partial[v][tile][in_tile];
    total *= scale;
    const int n = n0 + 16 * tile + j;
    const bool own = j < (tile ? own1 : own0);
    if (sizeof(OutT) == 2 && fusion.resid) {
        // One sum of squares per row and workgroup: the second tile's go through LDS to the first tile's threads.
        const float sq = stream_update(fusion, total, m, n, M, N, own);
        if (tile && j == 0) second_tile_sums[m] = sq;
        __syncthreads();
        if (!tile && j == 0 && m < M) fusion.square_sums_out[(size_t)m * gridDim.x + blockIdx.x] = sq + second_tile_sums[m];
        return;
    }
    if (m < M && own && n < N) y[(size_t)m * N + n] = (OutT)(fusion.bias ? total + fusion.bias[n] : total);
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

static int compute_units() {
    static int units = 0;
    if (!units) {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) == hipSuccess && hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
            units = prop.multiProcessorCount;
        else
            units = 256;
    }
    return units;
}

// ------------------------------------------------------------------------------------------
// 17 to 128 rows of activations.  Every slice of X is now as large as several tiles of W, so a
// workgroup whose wavefronts split K (each loading its own slice of X) would move several times
// more X than W.  Here the eight wavefronts of a workgroup take eight different tiles of W (128
// rows) over the same range of K instead, and share that range of X through LDS, a slab of 512 or
// 256 columns at a time; the ranges of K are spread over workgroups so that the chip is filled,
// and every workgroup writes its partial sums in float32, [split, M, N].  Adding them up is left
// to whoever reads the result next (the residual sum and norm that follow take partial sums),
// which costs no launch.
constexpr int SPLIT_TILE_ROWS = 16 * GEMM_WAVES;       // rows of W per workgroup
constexpr int SPLIT_MOST_ROWS = 128;                    // most rows of X
constexpr int SPLIT_AHEAD_FROM_SLABS = 4;               // slabs of 256 columns a workgroup from which W is asked for a slab ahead (beyond 64 rows)

// SLAB: columns of X staged at a time (512 up to 64 rows, 256 beyond: two slabs have to fit into LDS).
// GATED: W stacks a gate matrix on an up matrix ([N, K], gate rows first) and the result wanted is
// silu(x . gate^T) * (x . up^T) in bfloat16, [M, N / 2]: four wavefronts take 64 gate rows, the other four the up rows
// that belong to them, and the two halves meet in the epilogue; one range of K only (nothing is left to add up).
// AHEAD: the W of a slab is asked for a whole slab before it is met instead of half a slab.  With many rows of X a slab
// takes long to multiply, and a request made only half a slab ahead is waited for at every slab; it costs the registers
// of a second slab of W and a longer start, so it pays from four slabs a workgroup on (measured at 128 rows:
// 4096 x 12288 36.5 -> 33 us, 5120 x 25600 89 -> 73 us; two slabs a workgroup 16.2 -> 16.8 us).
template <int MT, int SLAB, bool GATED, bool AHEAD>
__global__ __launch_bounds__(GEMM_WAVES * 64) void gemm_split_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                     void* __restrict__ out, int M, int N, int K, int k_range) {
    constexpr int SPLIT_PITCH = SLAB * 2 + 16;          // bytes per staged row: 16 rows apart are 64 banks apart
    constexpr int SPLIT_CHUNK = SLAB / 64;              // k steps of W whose loads are issued together: half a slab
    extern __shared__ __attribute__((aligned(16))) unsigned char staged[];      // [2][16 MT][SPLIT_PITCH]
    constexpr int BUFFER = 16 * MT * SPLIT_PITCH;
    constexpr int PIECES = 16 * MT * (SLAB / 8) / (GEMM_WAVES * 64);      // 16-byte pieces of a slab per thread
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, quad = lane >> 4;
    const int n0 = GATED ? blockIdx.x * (SPLIT_TILE_ROWS / 2) + 16 * (wave & 3) : blockIdx.x * SPLIT_TILE_ROWS + 16 * wave;
    const int k_first = blockIdx.y * k_range, k_last = min(K, k_first + k_range);
    const int w_row = GATED ? (wave < 4 ? min(n0 + col, N / 2 - 1) : N / 2 + min(n0 + col, N / 2 - 1)) : min(n0 + col, N - 1);
    const bf16_t* wp = w + (size_t)w_row * K + 8 * quad;
    const int k_safe = K - 8;
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    struct Chunk { bf16x8 a[SPLIT_CHUNK]; };
    auto load_chunk = [&](Chunk& c, int k0) {
#pragma unroll
        for (int u = 0; u < SPLIT_CHUNK; ++u) c.a[u] = *reinterpret_cast<const bf16x8*>(wp + min(k0 + 32 * u + 8 * quad, k_safe) - 8 * quad);
    };
    // The operands of X for the next k step are read from LDS while the products of this one run.
    struct Operands { bf16x8 b[MT]; };
    auto read_operands = [&](Operands& o, const unsigned char* slab, int k_in_slab) {
#pragma unroll
        for (int t = 0; t < MT; ++t) o.b[t] = *reinterpret_cast<const bf16x8*>(slab + (16 * t + col) * SPLIT_PITCH + 2 * (k_in_slab + 8 * quad));
    };
    auto multiply_chunk = [&](const Chunk& c, int k0, const unsigned char* slab, int k_in_slab) {
        Operands even, odd;
        read_operands(even, slab, k_in_slab);
#pragma unroll
        for (int u = 0; u < SPLIT_CHUNK; ++u) {
            if (u + 1 < SPLIT_CHUNK) read_operands((u & 1) ? even : odd, slab, k_in_slab + 32 * (u + 1));
            const Operands& o = (u & 1) ? odd : even;
            bf16x8 a = c.a[u];
            if (k0 + 32 * u + 8 * quad >= k_last) a = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, o.b[t], acc[t], 0, 0, 0);
        }
    };
    // A slab of X: rows beyond M and columns beyond K are staged as zeros (their loads read a valid address).
    struct Slab { bf16x8 piece[PIECES]; };
    auto load_slab = [&](Slab& r, int k0) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int e = tid + GEMM_WAVES * 64 * j, m = e / (SLAB / 8), k = k0 + 8 * (e % (SLAB / 8));
            r.piece[j] = *reinterpret_cast<const bf16x8*>(x + (size_t)min(m, M - 1) * K + min(k, k_safe));
        }
    };
    auto store_slab = [&](const Slab& r, int k0, unsigned char* slab) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int e = tid + GEMM_WAVES * 64 * j, m = e / (SLAB / 8), piece = e % (SLAB / 8);
            bf16x8 v = r.piece[j];
            if (m >= M || k0 + 8 * piece >= K) v = (bf16x8){0, 0, 0, 0, 0, 0, 0, 0};
            *reinterpret_cast<bf16x8*>(slab + m * SPLIT_PITCH + 16 * piece) = v;
        }
    };
    constexpr int HALF = 32 * SPLIT_CHUNK;          // a slab is two chunks of W
    if (AHEAD && k_first < k_last) {
        // Every load of the loop is issued whether or not its slab exists (a slab past the last one is the last one again,
        // from cache): the number of loads in flight at each wait is then the same on every path, and no wait is for more
        // than it needs.
        const int n_slabs = (k_last - k_first + SLAB - 1) / SLAB, k_end = k_first + (n_slabs - 1) * SLAB;
        Chunk p0, q0, p1, q1;
        Slab next;
        load_slab(next, k_first);
        load_chunk(p0, k_first);
        load_chunk(q0, k_first + HALF);
        store_slab(next, k_first, staged);
        __syncthreads();
        load_chunk(p1, min(k_first + SLAB, k_end));
        load_chunk(q1, min(k_first + SLAB, k_end) + HALF);
        // The scheduler would move loads down to just before their use (fewer registers live): they stay where they are.
        __builtin_amdgcn_sched_barrier(0);
        int buffer = 0, k0 = k_first;
        // A slab that another follows: its successor's X travels through registers to the other buffer while it is
        // multiplied, and the W of the slab after that is asked for, a chunk as soon as the registers of one are free.
        auto slab_and_next = [&](Chunk& p, Chunk& q) {
            load_slab(next, k0 + SLAB);
            __builtin_amdgcn_sched_barrier(0);
            multiply_chunk(p, k0, staged + buffer * BUFFER, 0);
            load_chunk(p, min(k0 + 2 * SLAB, k_end));
            __builtin_amdgcn_sched_barrier(0);
            multiply_chunk(q, k0 + HALF, staged + buffer * BUFFER, HALF);
            load_chunk(q, min(k0 + 2 * SLAB, k_end) + HALF);
            __builtin_amdgcn_sched_barrier(0);
            store_slab(next, k0 + SLAB, staged + (buffer ^ 1) * BUFFER);
            __syncthreads();
            buffer ^= 1;
            k0 += SLAB;
        };
        int left = n_slabs;
        for (; left > 2; left -= 2) {
            slab_and_next(p0, q0);
            slab_and_next(p1, q1);
        }
        if (left == 2) {
            slab_and_next(p0, q0);
            multiply_chunk(p1, k0, staged + buffer * BUFFER, 0);
            multiply_chunk(q1, k0 + HALF, staged + buffer * BUFFER, HALF);
        } else {
            multiply_chunk(p0, k0, staged + buffer * BUFFER, 0);
            multiply_chunk(q0, k0 + HALF, staged + buffer * BUFFER, HALF);
        }
    } else if (k_first < k_last) {
        Chunk p, q;
        Slab next;
        // Loads are issued in the order in which they are waited for: X of a slab before the W it meets.
        load_slab(next, k_first);
        load_chunk(p, k_first);
        load_chunk(q, k_first + HALF);
        store_slab(next, k_first, staged);
        __syncthreads();
        int buffer = 0, k0 = k_first;
        // While a slab is multiplied, the next one travels through registers to the other buffer (which every
        // wavefront has finished reading before the barrier that ended the previous round) and the W it will
        // meet is requested, a chunk as soon as the registers of one are free.  The last slab requests nothing.
        for (; k0 + SLAB < k_last; k0 += SLAB, buffer ^= 1) {
            load_slab(next, k0 + SLAB);
            multiply_chunk(p, k0, staged + buffer * BUFFER, 0);
            load_chunk(p, k0 + SLAB);
            multiply_chunk(q, k0 + HALF, staged + buffer * BUFFER, HALF);
            load_chunk(q, k0 + SLAB + HALF);
            store_slab(next, k0 + SLAB, staged + (buffer ^ 1) * BUFFER);
            __syncthreads();
        }
        multiply_chunk(p, k0, staged + buffer * BUFFER, 0);
        multiply_chunk(q, k0 + HALF, staged + buffer * BUFFER, HALF);
    }
    // Lane (col, quad) holds Y[16 t + col][n0 + 4 quad .. + 4].
    if (GATED) {
        // The up halves go through LDS (the staged X is done with) to the wavefronts that hold their gate halves.
        const int half = N / 2;
        __syncthreads();
        f32x4* exchange = reinterpret_cast<f32x4*>(staged);            // [4 wavefronts][MT][64 lanes]
        if (wave >= 4) {
#pragma unroll
            for (int t = 0; t < MT; ++t) exchange[((wave - 4) * MT + t) * 64 + lane] = acc[t];
        }
        __syncthreads();
        if (wave >= 4) return;
        bf16_t* hidden = reinterpret_cast<bf16_t*>(out);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = 16 * t + col, n = n0 + 4 * quad;
            const f32x4 up = exchange[(wave * MT + t) * 64 + lane];
            if (m >= M) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float gate = acc[t][r];
                if (n + r < half) hidden[(size_t)m * half + n + r] = (bf16_t)(gate / (1.f + expf(-gate)) * up[r]);
            }
        }
        return;
    }
    float* partial = reinterpret_cast<float*>(out);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + col, n = n0 + 4 * quad;
        if (m >= M) continue;
        float* dst = partial + ((size_t)blockIdx.y * M + m) * N + n;
        if (n + 3 < N && N % 4 == 0) {
            *reinterpret_cast<f32x4*>(dst) = acc[t];
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n + r < N) dst[r] = acc[t][r];
        }
    }
}

// Columns of X per workgroup (a multiple of 256) for `tiles` workgroups per range of K: the one with which the compute units, working
// through the workgroups in rounds, are done soonest; a round costs its columns plus a fixed part.
static int split_range(long tiles, int K) {
    const int units = compute_units();
    const int whole = (K + 255) / 256 * 256;
    long best_cost = -1;
    int best = whole;
    for (int range = whole; range >= 256; range -= 256) {
        const long splits = (K + range - 1) / range;
        const long cost = (tiles * splits + units - 1) / units * (range + 512);
        if (best_cost < 0 || cost < best_cost) {       // ties: the larger range, fewer partial sums
            best_cost = cost;
            best = range;
        }
    }
    return best;
}


// Rows of W per workgroup.  The compute units work through the workgroups in rounds, a round takes
// as long as its workgroups have rows (plus a fixed part), and a round that is not full costs as
// much as a full one: so the best size is the one with the smallest rounds * (rows + fixed part).
// Up to 16 rows are one tile per wavefront, 17 to 32 two tiles, which halves the activations'
// share of what a workgroup loads (measured: worth 10 % at 9 to 16 rows of activations, 3 % at 4
// to 8, and a loss of as much below that, where the activations come from the first-level cache).
// GATED counts pairs of a gate row and an up row: one tile of 8 pairs, or two tiles of up to 16.
// `request`: 0 picks, otherwise the size to use (GATED: -1 for the one-tile form).
static int choose_rows(int M, int N, bool gated, int request) {
    const long total = gated ? N / 2 : N;
    const int units = compute_units();
    if (gated) {
        if (request == -1) return -1;
        if (request > 0) return request;
        long best_cost = ((total + 7) / 8 + units - 1) / units * 21;                 // one tile: 8 pairs + 2.5
        int best = -1;
        for (int r = 16; r >= 8; r -= 2) {
            const long cost = ((total + r - 1) / r + units - 1) / units * (2 * r + 4);   // two tiles: r pairs + 2
            if (cost < best_cost) {
                best_cost = cost;
                best = r;
            }
        }
        return best;
    }
    if (request > 0) return request;
    long best_cost = -1;
    int best = 16;
    for (int r = (M <= 16 ? 32 : 16); r >= 8; r -= 4) {
        long cost = ((total + r - 1) / r + units - 1) / units * (r + 4) * 100;
        if (r > 16 && M < 4) cost = cost * 115 / 100;
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = r;
        }
    }
    return best;
}

#define LSA_FOR_CHUNK(chunk, LAUNCH)   \
    switch (chunk) {                   \
        case 4: LAUNCH(4); break;      \
        case 5: LAUNCH(5); break;      \
        case 6: LAUNCH(6); break;      \
        case 7: LAUNCH(7); break;      \
        default: LAUNCH(8); break;     \
    }

// Workgroups and partial sums of squares per row (stream update) for a size.
static void layout(int N, bool gated, int rows, int* workgroups, int* parts) {
    const long total = gated ? N / 2 : N;
    const int r = rows == -1 ? 8 : rows;
    *workgroups = (int)((total + r - 1) / r);
    *parts = *workgroups;
}

template <typename OutT, bool GATED>
static int launch(const bf16_t* x, const bf16_t* w, OutT* y, int M, int N, int K, int rows, const Fusion& fusion, hipStream_t stream) {
    const dim3 block(GEMM_WAVES * 64);
    int workgroups, parts;
    layout(N, GATED, rows, &workgroups, &parts);
    const dim3 grid(workgroups);
    const bool two_tiles = GATED ? rows != -1 : rows > 16;
    if (two_tiles) {
        if (M > 16 || rows > (GATED ? 16 : 32)) return -1;
#define LSA_WIDE(CH) gemm_skinny_wide_kernel<OutT, GATED, CH><<<grid, block, 0, stream>>>(x, w, y, M, N, K, rows, fusion)
        LSA_FOR_CHUNK(best_chunk(K), LSA_WIDE)
#undef LSA_WIDE
        LSA_LAUNCH_CHECK();
    }
    if (rows < 1 && !GATED) return -1;
    if (M <= 16) {
#define LSA_ONE(CH) gemm_skinny_kernel<1, OutT, GATED, CH><<<grid, block, 0, stream>>>(x, w, y, M, N, K, rows, fusion)
        LSA_FOR_CHUNK(best_chunk(K), LSA_ONE)
#undef LSA_ONE
    } else if (GATED) {
        return -1;
    } else if (M <= 32) {
        gemm_skinny_kernel<2, OutT, false, 8><<<grid, block, 0, stream>>>(x, w, y, M, N, K, rows, fusion);
    } else {
        gemm_skinny_kernel<4, OutT, false, 4><<<grid, block, 0, stream>>>(x, w, y, M, N, K, rows, fusion);
    }
    LSA_LAUNCH_CHECK();
}

static bool fusion_fits(int M, const float* square_sums, int n_parts, const void* resid) {
    if (!square_sums && !resid) return true;
    if (M > FUSED_ROWS) return false;
    if (square_sums && (n_parts <= 0 || n_parts > (M <= GEMM_WAVES ? SCALE_PARTS : SCALE_PARTS / 2))) return false;
    return true;
}

// out_float32: 0 writes bfloat16, 1 writes float32.  rows: rows of W per workgroup, 1 to 32 (more than 16
// only for M <= 16), or 0 to let the size decide.  square_sums [M, n_parts] (or null) asks for the row scale
// rsqrt(sum / K + eps), M <= 16.  bias [N] (or null) is added to the sums before they are rounded.  Refuses
// (returns -1) what it cannot take.
LSA_EXPORT int lsa_gemm_skinny(int out_float32, const void* x, const void* w, void* y, int M, int N, int K, int rows,
                               const float* square_sums, int n_parts, float eps, const float* bias, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 != 0 || K < 8 || rows < 0 || rows > 32 || (rows > 16 && M > 16)) return -1;
    if (!fusion_fits(M, square_sums, n_parts, nullptr)) return -1;
    const Fusion fusion = {square_sums, n_parts, eps, nullptr, nullptr, nullptr, nullptr, nullptr, bias};
    rows = choose_rows(M, N, false, rows);
    return out_float32 ? launch<float, false>((const bf16_t*)x, (const bf16_t*)w, (float*)y, M, N, K, rows, fusion, stream)
                       : launch<bf16_t, false>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, M, N, K, rows, fusion, stream);
}

// Partial sums per row that lsa_gemm_skinny_stream writes for this size (the second dimension of square_sums_out).
LSA_EXPORT int lsa_gemm_skinny_parts(int M, int N, int rows) {
    if (M <= 0 || N <= 0 || rows < 0 || rows > 32) return -1;
    int workgroups, parts;
    layout(N, false, choose_rows(M, N, false, rows), &workgroups, &parts);
    return parts;
}

// The product as an update of a residual stream that a norm follows (see the top of the file), M <= 16:
//   resid_out = round(resid + round(x . w^T [/ rms, if square_sums])), weighted_out = round(resid_out * norm_weight),
//   square_sums_out [M, lsa_gemm_skinny_parts(M, N, rows)] = sums of resid_out^2 over the columns of each workgroup.
// resid_out may be resid itself.
LSA_EXPORT int lsa_gemm_skinny_stream(const void* x, const void* w, int M, int N, int K, int rows,
                                      const float* square_sums, int n_parts, float eps,
                                      const void* resid, const float* norm_weight, void* resid_out, void* weighted_out,
                                      float* square_sums_out, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 != 0 || K < 8 || rows < 0 || rows > 32 || !resid || !norm_weight || !resid_out || !weighted_out || !square_sums_out)
        return -1;
    if (!fusion_fits(M, square_sums, n_parts, resid)) return -1;
    const Fusion fusion = {square_sums, n_parts, eps, (const bf16_t*)resid, norm_weight, (bf16_t*)resid_out, (bf16_t*)weighted_out,
                           square_sums_out, nullptr};
    return launch<bf16_t, false>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)nullptr, M, N, K, choose_rows(M, N, false, rows), fusion, stream);
}

// hidden[M, I] = silu(x . gate^T) * (x . up^T) with gate_up [2I, K] (gate rows first); M <= 16, I a multiple of 8.
// rows: pairs of a gate and an up row per workgroup in the two-tile form, 1 to 16; -1: the one-tile form (8 pairs);
// 0 to let the size decide.  square_sums as in lsa_gemm_skinny.
LSA_EXPORT int lsa_gemm_skinny_gated(const void* x, const void* gate_up, void* hidden, int M, int I, int K, int rows,
                                     const float* square_sums, int n_parts, float eps, hipStream_t stream) {
    if (M <= 0 || I <= 0) return 0;
    if (M > 16 || K % 8 != 0 || K < 8 || I % 8 != 0 || rows < -1 || rows > 16) return -1;
    if (!fusion_fits(M, square_sums, n_parts, nullptr)) return -1;
    const Fusion fusion = {square_sums, n_parts, eps, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    return launch<bf16_t, true>((const bf16_t*)x, (const bf16_t*)gate_up, (bf16_t*)hidden, M, 2 * I, K, choose_rows(M, 2 * I, true, rows),
                                fusion, stream);
}

// Partial sums that lsa_gemm_split writes for a size (the first dimension of its result), or -1 if it does not
// take the size: M <= 128 (it is made for 17 and more, but on some shapes it beats the few-row kernel from 9 on),
// K a multiple of 8.
LSA_EXPORT int lsa_gemm_split_parts(int M, int N, int K) {
    if (M < 1 || M > SPLIT_MOST_ROWS || N <= 0 || K < 8 || K % 8 != 0) return -1;
    const int range = split_range((N + SPLIT_TILE_ROWS - 1) / SPLIT_TILE_ROWS, K);
    return (K + range - 1) / range;
}

// partial [lsa_gemm_split_parts(M, N, K), M, N] float32: sums over ranges of K of x [M, K] . w [N, K]^T (bfloat16);
// their sum over the first dimension is the product.
LSA_EXPORT int lsa_gemm_split(const void* x, const void* w, float* partial, int M, int N, int K, hipStream_t stream) {
    if (lsa_gemm_split_parts(M, N, K) < 0 || !x || !w || !partial) return -1;
    const int range = split_range((N + SPLIT_TILE_ROWS - 1) / SPLIT_TILE_ROWS, K);
    const dim3 grid((N + SPLIT_TILE_ROWS - 1) / SPLIT_TILE_ROWS, (K + range - 1) / range), block(GEMM_WAVES * 64);
    // More LDS than a kernel gets by default: asked for once per kernel and device.
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return -1;
#define LSA_SPLIT(MT, SLAB, GATED, AHEAD)                                                                                      \
    {                                                                                                                          \
        static bool sized[64] = {};                                                                                            \
        constexpr int bytes = 2 * 16 * MT * (2 * SLAB + 16);                                                                   \
        if (!sized[device]) {                                                                                                  \
            const hipError_t e = hipFuncSetAttribute((const void*)gemm_split_kernel<MT, SLAB, GATED, AHEAD>,                   \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, bytes);                       \
            if (e != hipSuccess) return (int)e;                                                                                \
            sized[device] = true;                                                                                              \
        }                                                                                                                      \
        gemm_split_kernel<MT, SLAB, GATED, AHEAD><<<grid, block, bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, out, M, N, K, range); \
    }
    // Slabs of 512 columns where two of them fit into LDS and the range is made of whole ones (a slab is loaded whole).
    const bool wide = range % 512 == 0;
    // Beyond 64 rows, W a whole slab ahead where a workgroup has four slabs or more (see the kernel).
    const bool ahead = ((range < K ? range : K) + 255) / 256 >= SPLIT_AHEAD_FROM_SLABS;
    void* out = partial;
    if (M <= 32) { if (wide) LSA_SPLIT(2, 512, false, false) else LSA_SPLIT(2, 256, false, false) }
    else if (M <= 48) { if (wide) LSA_SPLIT(3, 512, false, false) else LSA_SPLIT(3, 256, false, false) }
    else if (M <= 64) { if (wide) LSA_SPLIT(4, 512, false, false) else LSA_SPLIT(4, 256, false, false) }
    else if (M <= 96) { if (ahead) LSA_SPLIT(6, 256, false, true) else LSA_SPLIT(6, 256, false, false) }
    else { if (ahead) LSA_SPLIT(8, 256, false, true) else LSA_SPLIT(8, 256, false, false) }
    LSA_LAUNCH_CHECK();
}

constexpr int SPLIT_GATED_MOST_ROWS = 32;     // beyond, the library's product and the activation kernel are faster (measured)

// Whether lsa_gemm_split_gated takes a size: 17 <= M <= 32, K a multiple of 8, and so many pairs of a gate and an up
// row that one range of K per workgroup fills the chip (with ranges to add up there is no result to activate).
// Whether it is the faster way is for the caller to measure: with more rounds of workgroups than one the library
// has been seen to win (118 against 104 us at 400 workgroups).
LSA_EXPORT int lsa_gemm_split_gated_fits(int M, int I, int K) {
    if (M <= 16 || M > SPLIT_GATED_MOST_ROWS || I <= 0 || K < 8 || K % 8 != 0) return 0;
    return split_range((I + SPLIT_TILE_ROWS / 2 - 1) / (SPLIT_TILE_ROWS / 2), K) >= K ? 1 : 0;
}

// hidden [M, I] = silu(x . gate^T) * (x . up^T) in bfloat16, gate_up [2 I, K] with the gate rows first.
LSA_EXPORT int lsa_gemm_split_gated(const void* x, const void* w, void* hidden, int M, int I, int K, hipStream_t stream) {
    if (!lsa_gemm_split_gated_fits(M, I, K) || !x || !w || !hidden) return -1;
    const int N = 2 * I, range = (K + 255) / 256 * 256;
    const dim3 grid((I + SPLIT_TILE_ROWS / 2 - 1) / (SPLIT_TILE_ROWS / 2), 1), block(GEMM_WAVES * 64);
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return -1;
    void* out = hidden;
    const bool wide = range % 512 == 0;
    if (wide) LSA_SPLIT(2, 512, true, false) else LSA_SPLIT(2, 256, true, false)
#undef LSA_SPLIT
    LSA_LAUNCH_CHECK();
}
