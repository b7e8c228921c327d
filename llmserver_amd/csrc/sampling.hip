// Sampling from float32 logits, one block per row: greedy (temperature 0) takes the first
// maximum; otherwise the token is drawn from softmax(logits / temperature) by inverting the
// cumulative distribution at a uniform number the host supplies per row (so a request's
// tokens do not depend on what else is in the batch).  The maximum, the sum of exponentials and
// the running sums are 32-bit and walk the vocabulary in a fixed order.
#include "common.hpp"

using namespace lsa;

constexpr int SAMPLE_THREADS = 1024;
constexpr int SAMPLE_WAVES = SAMPLE_THREADS / 64;

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform, int* __restrict__ out, int vocab) {
    __shared__ float s_val[SAMPLE_WAVES];
    __shared__ int s_idx[SAMPLE_WAVES];
    __shared__ float s_sum[SAMPLE_WAVES];
    const float* x = logits + (size_t)blockIdx.x * vocab;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // Each wavefront owns a contiguous segment of the vocabulary (a multiple of 64 long).
    const int per_wave = ((vocab + SAMPLE_WAVES - 1) / SAMPLE_WAVES + 63) / 64 * 64;
    const int seg_begin = wave * per_wave, seg_end = min(vocab, seg_begin + per_wave);

    float best = -__builtin_huge_valf();
    int best_i = 0x7fffffff;
    for (int i = seg_begin + lane; i < seg_end; i += 64) {
        const float v = x[i];
        if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float ov = __shfl_xor(best, offset, 64);
        const int oi = __shfl_xor(best_i, offset, 64);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (lane == 0) { s_val[wave] = best; s_idx[wave] = best_i; }
    __syncthreads();
    best = s_val[0]; best_i = s_idx[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w)
        if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) { best = s_val[w]; best_i = s_idx[w]; }
    const float temp = temperature[blockIdx.x];
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
        return;
    }
    const float inv_temp = 1.f / temp;
    float part = 0.f;
    for (int i = seg_begin + lane; i < seg_end; i += 64) part += expf((x[i] - best) * inv_temp);
    part = wave_sum(part);
    if (lane == 0) s_sum[wave] = part;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) total += s_sum[w];
    const float target = uniform[blockIdx.x] * total;
    // The segment in which the running sum passes the target (the last non-empty one if rounding leaves none).
    float before = 0.f;
    int chosen = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (w * per_wave >= vocab) break;
        chosen = w;
        if (before + s_sum[w] > target) break;
        if ((w + 1) * per_wave < vocab) before += s_sum[w];
    }
    if (wave != chosen) return;
    int result = seg_end - 1;
    bool found = false;
    for (int base = seg_begin; base < seg_end && !found; base += 64) {
        const int i = base + lane;
        const float p = i < seg_end ? expf((x[i] - best) * inv_temp) : 0.f;
        float scan = p;                       // inclusive prefix sum over the 64 lanes
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const float up = __shfl_up(scan, offset, 64);
            if (lane >= offset) scan += up;
        }
        const bool hit = i < seg_end && before + scan > target;
        const unsigned long long mask = __ballot(hit);
        if (mask) {
            result = base + __builtin_ctzll(mask);
            found = true;
        }
        before += __shfl(scan, 63, 64);
    }
    if (lane == 0) out[blockIdx.x] = result;
}

LSA_EXPORT int lsa_sample(const float* logits, const float* temperature, const float* uniform, int* out, int n_rows, int vocab,
                          hipStream_t stream) {
    if (n_rows <= 0) return 0;
    sample_kernel<<<n_rows, SAMPLE_THREADS, 0, stream>>>(logits, temperature, uniform, out, vocab);
    LSA_LAUNCH_CHECK();
}
