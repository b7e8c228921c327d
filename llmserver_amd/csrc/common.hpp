// Shared helpers of the gfx950 kernels: element types, conversions, wavefront reductions.
// Wavefronts are 64 lanes wide; every reduction below is written for that width.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lsa {

typedef __bf16 bf16_t;

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int kVec = 4;                       // elements per 16-byte vector
    __device__ static inline float load(const float* p) { return *p; }
    __device__ static inline void store(float* p, float v) { *p = v; }
    __device__ static inline float round(float v) { return v; }
};
template <> struct Elem<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static inline float load(const bf16_t* p) { return (float)(*p); }
    __device__ static inline void store(bf16_t* p, float v) { *p = (bf16_t)v; }
    __device__ static inline float round(float v) { return (float)((bf16_t)v); }
};

// A 16-byte vector of T, loaded and stored as one transaction.
template <typename T> struct alignas(16) Vec16 {
    T v[Elem<T>::kVec];
};

template <typename T>
__device__ inline Vec16<T> load_vec16(const T* p) {
    return *reinterpret_cast<const Vec16<T>*>(p);
}
template <typename T>
__device__ inline void store_vec16(T* p, const Vec16<T>& x) {
    *reinterpret_cast<Vec16<T>*>(p) = x;
}

__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result. `scratch` holds 16 floats.
__device__ inline float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();                      // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[w];   // same order in every thread
    return total;
}

}  // namespace lsa

#define LSA_EXPORT extern "C" __attribute__((visibility("default")))
#define LSA_LAUNCH_CHECK() return (int)hipGetLastError()
