// Per-head q/k RMSNorm, rotate-half rotation and the write of new keys and values into their
// pages, for all tokens of the step (portions of prompts and decoded tokens alike).
//
// rotary_table: cos and sin of position * inv_freq for every token of the step, once per step
//   (the angles depend on the token and the pair of dimensions only, not on the layer or head).
// qk_norm_rope_kv_write: one wavefront per (token, head), four heads per workgroup.  q heads are
//   normalised, rotated and written back in place into the projection buffer; k heads are
//   normalised, rotated and stored at keys[page][kv_head][slot][:]; v heads are stored transposed
//   at values[page][kv_head][:][slot].  The page of a token is table[row][position / page_size];
//   nothing is allocated here.
// value_tiles: for long portions, the v heads go through LDS in tiles of 64 tokens so that the
//   transposed stores of neighbouring tokens (neighbouring slots of a page) coalesce.
// Norm sums, angles, cos/sin and the rotation are 32-bit; results are rounded once.
#include "common.hpp"

using namespace lsa;

__global__ void rotary_table_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                    float* __restrict__ cos_sin, int half, int n_tokens) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_tokens * half) return;
    const int token = i / half, pair = i % half;
    const float angle = (float)positions[token] * inv_freq[pair];
    cos_sin[(size_t)token * 2 * half + pair] = cosf(angle);
    cos_sin[(size_t)token * 2 * half + half + pair] = sinf(angle);
}

template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv,                 // [tokens, (Hq + 2 Hkv) * d]
    T* __restrict__ keys,                // [pages, Hkv, page_size, d]
    T* __restrict__ values,              // [pages, Hkv, d, page_size]
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ cos_sin,   // [tokens, d] (cos of the d/2 pairs, then sin) or nullptr
    int page_size, int n_q, int n_kv, int d, int write_cache, int n_heads) {
    const int token = blockIdx.x, head = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (head >= n_heads) return;
    const int half = d >> 1;
    const bool is_q = head < n_q, is_k = !is_q && head < n_q + n_kv;
    if (!is_q && !write_cache) return;
    T* src = qkv + (size_t)token * (n_q + 2 * n_kv) * d + (size_t)head * d;
    size_t page = 0;
    int slot = 0;
    if (!is_q) {
        const int pos = positions[token];
        const int p = table[(size_t)token_row[token] * table_stride + pos / page_size];
        if (p < 0) return;               // the host never schedules a token without a page
        page = (size_t)p;
        slot = pos % page_size;
    }
    if (!is_q && !is_k) {                // value head: copy, transposed
        T* dst = values + ((page * n_kv + (head - n_q - n_kv)) * d) * page_size + slot;
        for (int i = lane; i < d; i += 64) dst[(size_t)i * page_size] = src[i];
        return;
    }
    const float* w = is_q ? q_weight : k_weight;
    float rstd = 1.f;
    if (w) {
        float sq = 0.f;
        for (int i = lane; i < d; i += 64) {
            const float x = (float)src[i];
            sq += x * x;
        }
        rstd = rsqrtf(wave_sum(sq) / (float)d + eps);
    }
    T* dst = is_q ? src : keys + ((page * n_kv + (head - n_q)) * page_size + slot) * d;
    const float* cs = cos_sin ? cos_sin + (size_t)token * d : nullptr;
    for (int i = lane; i < half; i += 64) {
        float x1 = (float)src[i], x2 = (float)src[i + half];
        if (w) {
            x1 = x1 * rstd * w[i];
            x2 = x2 * rstd * w[i + half];
        }
        float r1 = x1, r2 = x2;
        if (cs) {
            const float c = cs[i], s = cs[half + i];
            r1 = x1 * c - x2 * s;
            r2 = x2 * c + x1 * s;
        }
        dst[i] = (T)r1;
        dst[i + half] = (T)r2;
    }
}

constexpr int VT_TOKENS = 64;

template <typename T>
__global__ __launch_bounds__(256) void value_tiles_kernel(
    const T* __restrict__ qkv, T* __restrict__ values, const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions, int page_size, int n_q, int n_kv, int d, int n_tokens) {
    extern __shared__ unsigned char tile_bytes[];          // [VT_TOKENS][d + 2] elements of T
    T* tile = reinterpret_cast<T*>(tile_bytes);
    const int token0 = blockIdx.x * VT_TOKENS, kv_head = blockIdx.y;
    const int pitch = d + 2;
    const int width = (n_q + 2 * n_kv) * d;
    for (int e = threadIdx.x; e < VT_TOKENS * d; e += 256) {       // rows of the projection: coalesced over the head's d values
        const int t = e / d, i = e % d;
        if (token0 + t < n_tokens) tile[t * pitch + i] = qkv[(size_t)(token0 + t) * width + (size_t)(n_q + n_kv + kv_head) * d + i];
    }
    __syncthreads();
    const int t = threadIdx.x & (VT_TOKENS - 1);                   // this thread's token: neighbours write neighbouring slots
    const int token = token0 + t;
    if (token >= n_tokens) return;
    const int pos = positions[token];
    const int p = table[(size_t)token_row[token] * table_stride + pos / page_size];
    if (p < 0) return;
    T* dst = values + (((size_t)p * n_kv + kv_head) * d) * page_size + pos % page_size;
    for (int i = threadIdx.x / VT_TOKENS; i < d; i += 256 / VT_TOKENS) dst[(size_t)i * page_size] = tile[t * pitch + i];
}

template <typename T>
static int launch(void* qkv, void* keys, void* values, const int* table, int table_stride, const int* token_row,
                  const int* positions, const float* q_weight, const float* k_weight, float eps, const float* cos_sin,
                  int page_size, int n_q, int n_kv, int d, int write_cache, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    // Long portions: the v heads take the tiled path, the main kernel then covers q and k heads only.
    const bool tiled_values = write_cache && n_tokens >= 4 * VT_TOKENS;
    const int n_heads = tiled_values ? n_q + n_kv : n_q + 2 * n_kv;
    dim3 grid(n_tokens, (n_heads + 3) / 4);
    qk_norm_rope_kv_write_kernel<T><<<grid, 256, 0, stream>>>((T*)qkv, (T*)keys, (T*)values, table, table_stride, token_row,
                                                              positions, q_weight, k_weight, eps, cos_sin, page_size,
                                                              n_q, n_kv, d, write_cache, n_heads);
    int err = (int)hipGetLastError();
    if (err || !tiled_values) return err;
    dim3 vgrid((n_tokens + VT_TOKENS - 1) / VT_TOKENS, n_kv);
    value_tiles_kernel<T><<<vgrid, 256, VT_TOKENS * (d + 2) * sizeof(T), stream>>>((const T*)qkv, (T*)values, table, table_stride,
                                                                                  token_row, positions, page_size, n_q, n_kv, d, n_tokens);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_rotary_table(const int* positions, const float* inv_freq, float* cos_sin, int half, int n_tokens, hipStream_t stream) {
    const int total = n_tokens * half;
    if (total <= 0) return 0;
    rotary_table_kernel<<<(total + 255) / 256, 256, 0, stream>>>(positions, inv_freq, cos_sin, half, n_tokens);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_qk_norm_rope_kv_write(int dtype, void* qkv, void* keys, void* values, const int* table, int table_stride,
                                         const int* token_row, const int* positions, const float* q_weight,
                                         const float* k_weight, float eps, const float* cos_sin, int page_size, int n_q,
                                         int n_kv, int d, int write_cache, int n_tokens, hipStream_t stream) {
    return dtype ? launch<bf16_t>(qkv, keys, values, table, table_stride, token_row, positions, q_weight, k_weight, eps,
                                  cos_sin, page_size, n_q, n_kv, d, write_cache, n_tokens, stream)
                 : launch<float>(qkv, keys, values, table, table_stride, token_row, positions, q_weight, k_weight, eps,
                                 cos_sin, page_size, n_q, n_kv, d, write_cache, n_tokens, stream);
}
