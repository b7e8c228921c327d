// Sampling from float32 logits: greedy (temperature 0) takes the first maximum; otherwise the
// token is drawn from softmax(logits / temperature) by inverting the cumulative distribution at a
// uniform number the host supplies per row (so a request's tokens do not depend on what else is
// in the batch).  Two kernels: the first cuts every row into up to 64 contiguous chunks and
// finds each chunk's maximum, first position of it, and sum of exponentials; the second merges a
// row's chunks, finds the chunk in which the running sum passes the target and walks only that
// chunk.  Maximum, sums and running sums are 32-bit and walk the vocabulary in a fixed order.
#include "common.hpp"
#include "sampling.h"

#include <mutex>

using namespace lsa;

constexpr int MAX_CHUNKS = 64;
constexpr float MINUS_INF = -__builtin_huge_valf();

struct ChunkStat { float top; int first; float sum; int pad; };

__device__ inline void better(float& top, int& first, float other_top, int other_first) {
    if (other_top > top || (other_top == top && other_first < first)) { top = other_top; first = other_first; }
}

__global__ __launch_bounds__(256) void sample_chunks_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                            ChunkStat* __restrict__ stats, int vocab, int chunk_len) {
    __shared__ float s_top[4];
    __shared__ int s_first[4];
    __shared__ float s_sum[4];
    const int row = blockIdx.x, chunk = blockIdx.y;
    const float* x = logits + (size_t)row * vocab;
    const int begin = chunk * chunk_len, end = min(vocab, begin + chunk_len);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float top = MINUS_INF;
    int first = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += 256) better(top, first, x[i], i);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) better(top, first, __shfl_xor(top, offset, 64), __shfl_xor(first, offset, 64));
    if (lane == 0) { s_top[wave] = top; s_first[wave] = first; }
    __syncthreads();
    top = s_top[0]; first = s_first[0];
    for (int w = 1; w < 4; ++w) better(top, first, s_top[w], s_first[w]);
    const float temp = temperature[row];
    float total = 0.f;
    if (temp > 0.f && top > MINUS_INF) {
        const float inv_temp = 1.f / temp;
        // Fixed order: the chunk in groups of 64 consecutive tokens, a wavefront per group in turn.
        float part = 0.f;
        for (int base = begin + 64 * wave; base < end; base += 256) {
            const int i = base + lane;
            part += i < end ? expf((x[i] - top) * inv_temp) : 0.f;
        }
        part = wave_sum(part);
        if (lane == 0) s_sum[wave] = part;
        __syncthreads();
        total = s_sum[0] + s_sum[1] + s_sum[2] + s_sum[3];
    }
    if (threadIdx.x == 0) stats[(size_t)row * gridDim.y + chunk] = ChunkStat{top, first, total, 0};
}

__global__ __launch_bounds__(64) void sample_pick_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                         const float* __restrict__ uniform, const ChunkStat* __restrict__ stats,
                                                         int* __restrict__ out, int vocab, int chunk_len, int chunks) {
    const int row = blockIdx.x, lane = threadIdx.x;
    const ChunkStat mine = lane < chunks ? stats[(size_t)row * chunks + lane] : ChunkStat{MINUS_INF, 0x7fffffff, 0.f, 0};
    float top = mine.top;
    int first = mine.first;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) better(top, first, __shfl_xor(top, offset, 64), __shfl_xor(first, offset, 64));
    const float temp = temperature[row];
    if (!(temp > 0.f) || !(top > MINUS_INF)) {
        if (lane == 0) out[row] = first == 0x7fffffff ? 0 : first;
        return;
    }
    const float inv_temp = 1.f / temp;
    // Each chunk's sum, rescaled from its own maximum to the row's; inclusive running sums over the chunks.
    const float scaled = mine.top > MINUS_INF ? mine.sum * expf((mine.top - top) * inv_temp) : 0.f;
    float running = scaled;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
        const float up = __shfl_up(running, offset, 64);
        if (lane >= offset) running += up;
    }
    const float total = __shfl(running, 63, 64);
    const float target = uniform[row] * total;
    const unsigned long long passed = __ballot(lane < chunks && running > target);
    const int chunk = passed ? __builtin_ctzll(passed) : chunks - 1;          // rounding may leave none: the last chunk
    float before = __shfl(running - scaled, chunk, 64);
    const float* x = logits + (size_t)row * vocab;
    const int begin = chunk * chunk_len, end = min(vocab, begin + chunk_len);
    int result = end - 1;
    bool found = false;
    for (int base = begin; base < end && !found; base += 64) {
        const int i = base + lane;
        const float p = i < end ? expf((x[i] - top) * inv_temp) : 0.f;
        float scan = p;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const float up = __shfl_up(scan, offset, 64);
            if (lane >= offset) scan += up;
        }
        const unsigned long long hit = __ballot(i < end && before + scan > target);
        if (hit) {
            result = base + __builtin_ctzll(hit);
            found = true;
        }
        before += __shfl(scan, 63, 64);
    }
    if (lane == 0) out[row] = result;
}

LSA_EXPORT int lsa_sample_chunks(int vocab) {
    int chunks = (vocab + 2047) / 2048;
    return chunks < 1 ? 1 : (chunks > MAX_CHUNKS ? MAX_CHUNKS : chunks);
}

// workspace: n_rows * lsa_sample_chunks(vocab) * 16 bytes
LSA_EXPORT int lsa_sample(const float* logits, const float* temperature, const float* uniform, int* out, void* workspace, int n_rows,
                          int vocab, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    const int chunks = lsa_sample_chunks(vocab);
    const int chunk_len = ((vocab + chunks - 1) / chunks + 63) / 64 * 64;
    sample_chunks_kernel<<<dim3(n_rows, chunks), 256, 0, stream>>>(logits, temperature, (ChunkStat*)workspace, vocab, chunk_len);
    int err = (int)hipGetLastError();
    if (err) return err;
    sample_pick_kernel<<<n_rows, 64, 0, stream>>>(logits, temperature, uniform, (const ChunkStat*)workspace, out, vocab, chunk_len, chunks);
    LSA_LAUNCH_CHECK();
}

// ---- the variant that allocates nothing (declared and described in sampling.h) ----
static __device__ __align__(256) unsigned char scratch[(size_t)LSA_SAMPLE_STATIC_MAX_ROWS * MAX_CHUNKS * sizeof(ChunkStat)];

constexpr int MOST_DEVICES = 64;

// The address of `scratch` on the current device.  In host code the array's name is only a handle for this lookup,
// never a device address; every GPU has its own copy at its own address, so the answer is kept per device.
static int static_scratch(void** address) {
    static std::mutex guard;
    static void* known[MOST_DEVICES] = {};
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) return (int)status;
    if (device < 0 || device >= MOST_DEVICES) return LSA_SAMPLE_STATIC_BAD_DEVICE;
    std::lock_guard<std::mutex> lock(guard);
    if (known[device] == nullptr) {
        void* found = nullptr;
        status = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if (status != hipSuccess) return (int)status;
        if (found == nullptr) return (int)hipErrorInvalidSymbol;
        known[device] = found;
    }
    *address = known[device];
    return 0;
}

LSA_EXPORT int lsa_sample_static_max_rows(void) { return LSA_SAMPLE_STATIC_MAX_ROWS; }

LSA_EXPORT const char* lsa_sample_static_error(int code) {
    switch (code) {
        case 0: return "no error";
        case LSA_SAMPLE_STATIC_TOO_MANY_ROWS: return "lsa_sample_static takes at most 1024 rows a call (its fixed scratch array holds no more)";
        case LSA_SAMPLE_STATIC_BAD_DEVICE: return "lsa_sample_static: the current device's index is outside the table of scratch addresses";
        default: return hipGetErrorString((hipError_t)code);
    }
}

LSA_EXPORT int lsa_sample_static(const float* logits, const float* temperature, const float* uniform, int* out, int n_rows,
                                 int vocab, hipStream_t stream) {
    if (n_rows <= 0) return 0;
    if (n_rows > LSA_SAMPLE_STATIC_MAX_ROWS) return LSA_SAMPLE_STATIC_TOO_MANY_ROWS;
    void* stats = nullptr;
    const int status = static_scratch(&stats);
    if (status) return status;
    // Every (row, chunk) entry that the second kernel reads is written by the first: nothing of an earlier call is seen.
    return lsa_sample(logits, temperature, uniform, out, stats, n_rows, vocab, stream);
}
