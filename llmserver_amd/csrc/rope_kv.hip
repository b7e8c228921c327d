// Per-head q/k RMSNorm, rotate-half rotation and the write of new keys and values into their
// pages, for all tokens of the step (portions of prompts and decoded tokens alike).
//
// rotary_table: cos and sin of position * inv_freq for every token of the step, once per step
//   (the angles depend on the token and the pair of dimensions only, not on the layer or head).
// qk_norm_rope_kv_write: d / 16 lanes per (token, head), vector accesses throughout.  q heads are
//   normalised, rotated and written back in place into the projection buffer; k heads are
//   normalised, rotated and stored at keys[page][kv_head][slot][:]; v heads are stored transposed
//   at values[page][kv_head][:][slot].  The page of a token is table[row][position / page_size];
//   nothing is allocated here.
//   For long portions, the v heads go through LDS in tiles of 64 tokens so that the transposed stores of
//   neighbouring tokens (neighbouring slots of a page) coalesce: further workgroups of the same launch.
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

// A (token, head) pair is handled by d / 16 neighbouring lanes: lane j of them owns dimensions
// [8j, 8j + 8) of the first half and their rotation partners [d/2 + 8j, d/2 + 8j + 8), both as one
// vector load, so a wavefront covers 64 / (d / 16) pairs at once and every access is 16 bytes or more.
template <typename T> struct Eight {
    float v[8];
};
template <typename T>
__device__ inline Eight<T> load8(const T* p) {
    Eight<T> r;
    if (sizeof(T) == 2) {
        const Vec16<T> x = load_vec16(p);
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = (float)x.v[e];
    } else {
        const Vec16<T> x = load_vec16(p), y = load_vec16(p + 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            r.v[e] = (float)x.v[e];
            r.v[4 + e] = (float)y.v[e];
        }
    }
    return r;
}
template <typename T>
__device__ inline void store8(T* p, const float (&v)[8]) {
    if (sizeof(T) == 2) {
        Vec16<T> x;
#pragma unroll
        for (int e = 0; e < 8; ++e) x.v[e] = (T)v[e];
        store_vec16(p, x);
    } else {
        Vec16<T> x, y;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            x.v[e] = (T)v[e];
            y.v[e] = (T)v[4 + e];
        }
        store_vec16(p, x);
        store_vec16(p + 4, y);
    }
}

template <typename T>
__device__ __forceinline__ void qk_norm_rope_kv_write_block(
    const int block,
    T* __restrict__ qkv,                 // [tokens, (Hq + 2 Hkv) * d]
    T* __restrict__ keys,                // [pages, Hkv, page_size, d]
    T* __restrict__ values,              // [pages, Hkv, d, page_size]
    const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ cos_sin,   // [tokens, d] (cos of the d/2 pairs, then sin) or nullptr
    int page_size, int n_q, int n_kv, int d, int write_cache, int n_heads, int n_tokens) {
    const int lanes_per_pair = d >> 4, pairs_per_wave = 64 / lanes_per_pair;
    const int lane = threadIdx.x & 63, wave = block * 4 + (threadIdx.x >> 6);
    const int slot_in_wave = lane / lanes_per_pair, j = lane % lanes_per_pair;
    const long pair = (long)wave * pairs_per_wave + slot_in_wave;
    const bool active = slot_in_wave < pairs_per_wave && pair < (long)n_tokens * n_heads;
    const int token = active ? (int)(pair / n_heads) : 0, head = active ? (int)(pair % n_heads) : 0;
    const int half = d >> 1;
    const bool is_q = head < n_q, is_k = !is_q && head < n_q + n_kv;
    T* src = qkv + (size_t)token * (n_q + 2 * n_kv) * d + (size_t)head * d;
    const Eight<T> lo = load8(src + 8 * j), hi = load8(src + half + 8 * j);
    // Sum of squares of the head over its lanes (every lane of the wavefront takes part in the shuffles).
    float sq = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sq += lo.v[e] * lo.v[e] + hi.v[e] * hi.v[e];
    float total = 0.f;
    const int first_lane = lane - j;
    for (int other = 0; other < lanes_per_pair; ++other) total += __shfl(sq, first_lane + other, 64);
    if (!active || (!is_q && !write_cache)) return;
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
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            dst[(size_t)(8 * j + e) * page_size] = (T)lo.v[e];
            dst[(size_t)(half + 8 * j + e) * page_size] = (T)hi.v[e];
        }
        return;
    }
    const float* w = is_q ? q_weight : k_weight;
    float x1[8], x2[8];
    if (w) {
        const float rstd = rsqrtf(total / (float)d + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x1[e] = lo.v[e] * rstd * w[8 * j + e];
            x2[e] = hi.v[e] * rstd * w[half + 8 * j + e];
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x1[e] = lo.v[e];
            x2[e] = hi.v[e];
        }
    }
    if (cos_sin) {
        const float* cs = cos_sin + (size_t)token * d + 8 * j;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float c = cs[e], s = cs[half + e];
            const float r1 = x1[e] * c - x2[e] * s, r2 = x2[e] * c + x1[e] * s;
            x1[e] = r1;
            x2[e] = r2;
        }
    }
    T* dst = is_q ? src : keys + ((page * n_kv + (head - n_q)) * page_size + slot) * d;
    store8(dst + 8 * j, x1);
    store8(dst + half + 8 * j, x2);
}

constexpr int VT_TOKENS = 64;

// Values of long portions: a workgroup takes 64 consecutive tokens of one KV head through LDS, reads
// them from the projection in 16-byte pieces and writes them transposed, four slots of one
// dimension at a time (8 or 16 bytes) where four tokens are neighbours in one page, which is the
// rule inside a portion; a page's [d][page_size] block is contiguous, so these stores coalesce.
template <typename T>
__device__ __forceinline__ void value_tiles_block(
    const int tile_index, const int kv_head, unsigned char* tile_bytes,          // tile_bytes: [VT_TOKENS][d + VEC] elements of T in LDS
    const T* __restrict__ qkv, T* __restrict__ values, const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions, int page_size, int n_q, int n_kv, int d, int n_tokens) {
    constexpr int VEC = Elem<T>::kVec;
    __shared__ long group_base[VT_TOKENS / 4];             // element offset of the group's first slot in `values`, or -1
    __shared__ unsigned char covered[VT_TOKENS];           // token goes out with its group
    T* tile = reinterpret_cast<T*>(tile_bytes);
    const int token0 = tile_index * VT_TOKENS;
    const int pitch = d + VEC;
    const int width = (n_q + 2 * n_kv) * d;
    const int pieces = d / VEC;
    for (int e = threadIdx.x; e < VT_TOKENS * pieces; e += 256) {
        const int t = e / pieces, part = e % pieces;
        if (token0 + t < n_tokens)
            store_vec16(tile + t * pitch + part * VEC,
                        load_vec16(qkv + (size_t)(token0 + t) * width + (size_t)(n_q + n_kv + kv_head) * d + part * VEC));
    }
    // Four tokens go out together if they are one request's neighbours starting at a position that is a multiple
    // of four; the groups are laid so that this holds when the tile lies inside one portion.
    const int shift = (4 - (positions[min(token0, n_tokens - 1)] & 3)) & 3;
    if (threadIdx.x < VT_TOKENS) covered[threadIdx.x] = 0;
    __syncthreads();
    if (threadIdx.x < VT_TOKENS / 4) {
        const int local = shift + 4 * threadIdx.x, first = token0 + local;
        long base = -1;
        if (local + 3 < VT_TOKENS && first + 3 < n_tokens) {
            const int row = token_row[first], pos = positions[first];
            bool together = (pos & 3) == 0;
            for (int r = 1; r < 4; ++r) together = together && token_row[first + r] == row && positions[first + r] == pos + r;
            const int p = table[(size_t)row * table_stride + pos / page_size];
            if (together && p >= 0) {
                base = (((long)p * n_kv + kv_head) * d) * page_size + pos % page_size;
                for (int r = 0; r < 4; ++r) covered[local + r] = 1;
            }
        }
        group_base[threadIdx.x] = base;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < (VT_TOKENS / 4) * d; e += 256) {
        const int g = e & (VT_TOKENS / 4 - 1), i = e / (VT_TOKENS / 4);      // neighbouring threads: neighbouring groups of slots
        const long base = group_base[g];
        if (base < 0) continue;
        T four[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) four[r] = tile[(shift + 4 * g + r) * pitch + i];
        T* dst = values + base + (size_t)i * page_size;
        if (sizeof(T) == 2) *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<const uint2*>(four);
        else *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(four);
    }
    for (int e = threadIdx.x; e < VT_TOKENS * d; e += 256) {                  // the tokens that are in no such group
        const int t = e & (VT_TOKENS - 1), i = e / VT_TOKENS;
        const int token = token0 + t;
        if (covered[t] || token >= n_tokens) continue;
        const int pos = positions[token];
        const int p = table[(size_t)token_row[token] * table_stride + pos / page_size];
        if (p >= 0) values[(((size_t)p * n_kv + kv_head) * d + i) * page_size + pos % page_size] = tile[t * pitch + i];
    }
}

// One launch for both: the first `qk_blocks` workgroups take the (token, head) pairs of the q and k heads (and of the v
// heads, unless these go in tiles), the others a tile of 64 tokens of one KV head's values each.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_write_kernel(
    T* __restrict__ qkv, T* __restrict__ keys, T* __restrict__ values, const int* __restrict__ table, int table_stride,
    const int* __restrict__ token_row, const int* __restrict__ positions, const float* __restrict__ q_weight,
    const float* __restrict__ k_weight, float eps, const float* __restrict__ cos_sin, int page_size, int n_q, int n_kv, int d,
    int write_cache, int n_heads, int n_tokens, int qk_blocks) {
    extern __shared__ unsigned char tile_bytes[];          // (none unless values go in tiles)
    if ((int)blockIdx.x < qk_blocks) {
        qk_norm_rope_kv_write_block<T>((int)blockIdx.x, qkv, keys, values, table, table_stride, token_row, positions, q_weight, k_weight, eps,
                                       cos_sin, page_size, n_q, n_kv, d, write_cache, n_heads, n_tokens);
        return;
    }
    const int tile = ((int)blockIdx.x - qk_blocks) / n_kv, kv_head = ((int)blockIdx.x - qk_blocks) % n_kv;
    value_tiles_block<T>(tile, kv_head, tile_bytes, qkv, values, table, table_stride, token_row, positions, page_size, n_q, n_kv, d, n_tokens);
}

template <typename T>
static int launch(void* qkv, void* keys, void* values, const int* table, int table_stride, const int* token_row,
                  const int* positions, const float* q_weight, const float* k_weight, float eps, const float* cos_sin,
                  int page_size, int n_q, int n_kv, int d, int write_cache, int n_tokens, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    // Long portions: the v heads take the tiled path, the main kernel then covers q and k heads only.
    const bool tiled_values = write_cache && n_tokens >= 4 * VT_TOKENS;
    const int n_heads = tiled_values ? n_q + n_kv : n_q + 2 * n_kv;
    if (d % 16 != 0 || d > 1024) return -1;
    const long pairs = (long)n_tokens * n_heads;
    const int pairs_per_block = 4 * (64 / (d / 16));
    const long qk_blocks = (pairs + pairs_per_block - 1) / pairs_per_block;
    const long value_blocks = tiled_values ? (long)((n_tokens + VT_TOKENS - 1) / VT_TOKENS) * n_kv : 0;
    if (qk_blocks + value_blocks > 0x7fffffffL) return -1;
    const size_t tile_bytes = tiled_values ? (size_t)VT_TOKENS * (d + Elem<T>::kVec) * sizeof(T) : 0;
    qk_norm_rope_kv_write_kernel<T><<<dim3((unsigned)(qk_blocks + value_blocks)), 256, tile_bytes, stream>>>(
        (T*)qkv, (T*)keys, (T*)values, table, table_stride, token_row, positions, q_weight, k_weight, eps, cos_sin, page_size,
        n_q, n_kv, d, write_cache, n_heads, n_tokens, (int)qk_blocks);
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
