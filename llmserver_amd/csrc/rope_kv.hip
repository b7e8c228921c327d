// Per-head q/k RMSNorm, rotate-half rotation and the write of new keys and values into their
// pages, in one kernel over all tokens of the step (portions of prompts and decoded tokens alike).
//
// One wavefront per (token, head).  q heads are normalised, rotated and written back in place
// into the projection buffer; k heads are normalised, rotated and stored at
// keys[page][kv_head][slot][:]; v heads are stored transposed at values[page][kv_head][:][slot].
// The page of a token is table[row][position / page_size]; nothing is allocated here.
// Norm sums, angles, cos/sin and the rotation are 32-bit; results are rounded once.
#include "common.hpp"

using namespace lsa;

template <typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv,                 // [tokens, (Hq + 2 Hkv) * d]
    T* __restrict__ keys,                // [pages, Hkv, page_size, d]
    T* __restrict__ values,              // [pages, Hkv, d, page_size]
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ inv_freq,  // [d / 2] or nullptr
    int page_size, int n_q, int n_kv, int d, int write_cache) {
    const int token = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int half = d >> 1;
    const bool is_q = head < n_q, is_k = !is_q && head < n_q + n_kv;
    if (!is_q && !write_cache) return;
    T* src = qkv + (size_t)token * (n_q + 2 * n_kv) * d + (size_t)head * d;
    const int pos = positions[token];
    size_t page = 0;
    int slot = 0;
    if (!is_q) {
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
    float sq = 0.f;
    for (int i = lane; i < d; i += 64) {
        const float x = (float)src[i];
        sq += x * x;
    }
    float rstd = 1.f;
    if (w) rstd = rsqrtf(wave_sum(sq) / (float)d + eps);
    T* dst = is_q ? src : keys + ((page * n_kv + (head - n_q)) * page_size + slot) * d;
    for (int i = lane; i < half; i += 64) {
        float x1 = (float)src[i], x2 = (float)src[i + half];
        if (w) {
            x1 = x1 * rstd * w[i];
            x2 = x2 * rstd * w[i + half];
        }
        float r1 = x1, r2 = x2;
        if (inv_freq) {
            const float angle = (float)pos * inv_freq[i];
            const float c = cosf(angle), s = sinf(angle);
            r1 = x1 * c - x2 * s;
            r2 = x2 * c + x1 * s;
        }
        dst[i] = (T)r1;
        dst[i + half] = (T)r2;
    }
}

template <typename T>
static int launch(void* qkv, void* keys, void* values, const int* table, int table_stride, const int* token_row,
                  const int* positions, const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
                  int page_size, int n_q, int n_kv, int d, int write_cache, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    dim3 grid(n_tokens, n_q + 2 * n_kv);
    qk_norm_rope_kv_write_kernel<T><<<grid, 64, 0, stream>>>((T*)qkv, (T*)keys, (T*)values, table, table_stride, token_row,
                                                             positions, q_weight, k_weight, eps, inv_freq, page_size,
                                                             n_q, n_kv, d, write_cache);
    LSA_LAUNCH_CHECK();
}

LSA_EXPORT int lsa_qk_norm_rope_kv_write(int dtype, void* qkv, void* keys, void* values, const int* table, int table_stride,
                                         const int* token_row, const int* positions, const float* q_weight,
                                         const float* k_weight, float eps, const float* inv_freq, int page_size, int n_q,
                                         int n_kv, int d, int write_cache, int n_tokens, hipStream_t stream) {
    return dtype ? launch<bf16_t>(qkv, keys, values, table, table_stride, token_row, positions, q_weight, k_weight, eps,
                                  inv_freq, page_size, n_q, n_kv, d, write_cache, n_tokens, stream)
                 : launch<float>(qkv, keys, values, table, table_stride, token_row, positions, q_weight, k_weight, eps,
                                 inv_freq, page_size, n_q, n_kv, d, write_cache, n_tokens, stream);
}
