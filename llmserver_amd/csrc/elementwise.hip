// Row-wise kernels of the step: embedding lookup, residual sum fused with RMSNorm, SwiGLU,
// bias add.  One source for bfloat16 and float32 activations; sums, square sums, rsqrt,
// sigmoid and products are 32-bit inside, results are rounded once when stored.
#include "common.hpp"

using namespace lsa;

// ------------------------------------------------------------------------------------------
// Embedding: out[t, :] = table[ids[t], :].  An id outside the table gives a zero row (the
// host refuses such ids before the launch; the guard keeps a bad id from faulting the GPU).
template <typename T, bool VEC>
__global__ void embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids, T* __restrict__ out,
                                 int width, int vocab) {
    const int t = blockIdx.x;
    const int id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    const T* src = table + (size_t)(ok ? id : 0) * width;
    T* dst = out + (size_t)t * width;
    if (VEC) {
        constexpr int V = Elem<T>::kVec;
        for (int i = threadIdx.x * V; i < width; i += blockDim.x * V) {
            Vec16<T> x = load_vec16(src + i);
            if (!ok) {
#pragma unroll
                for (int k = 0; k < V; ++k) x.v[k] = (T)0.f;
            }
            store_vec16(dst + i, x);
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = ok ? src[i] : (T)0.f;
    }
}

// ------------------------------------------------------------------------------------------
// s = resid + delta (32-bit sum, rounded to T as the new residual stream);
// out = s * rsqrt(mean(s^2) + eps) * w, computed from the rounded s.
// rows == nullptr: every token row t: resid[t] = s, out[t] = norm.
// rows != nullptr: out[i] = norm of row rows[i]; resid is not written.
// The update of a row comes as `d` (values of the row's type) or as `parts` partial sums in float32 (`sums`, the
// same element of each `sums_stride` elements apart), which are added up and rounded to the row's type first.
struct PartialSums {
    const float* sums;
    int parts;
    size_t stride;
};

template <typename T, int V, bool PARTIAL>
__device__ inline void load_sum(const T* __restrict__ x, const T* __restrict__ d, const PartialSums& p, size_t row_offset, int i,
                                float (&s)[V]) {
    float update[V];
    const bool any = PARTIAL || d;
    if (PARTIAL) {
#pragma unroll
        for (int k = 0; k < V; ++k) update[k] = 0.f;
        const float* src = p.sums + row_offset + i;
        if (V % 4 == 0) {
            // Four parts' loads are issued together: the parts are read in a quarter of the trips to memory.
            constexpr int Q = V % 4 == 0 ? V / 4 : 1;
            int part = 0;
            for (; part + 4 <= p.parts; part += 4, src += 4 * p.stride) {
                float4 v[4][Q];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int k = 0; k < Q; ++k) v[j][k] = *reinterpret_cast<const float4*>(src + j * p.stride + 4 * k);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int k = 0; k < Q; ++k) {
                        update[4 * k] += v[j][k].x;
                        update[4 * k + 1] += v[j][k].y;
                        update[4 * k + 2] += v[j][k].z;
                        update[4 * k + 3] += v[j][k].w;
                    }
            }
            for (; part < p.parts; ++part, src += p.stride) {
#pragma unroll
                for (int k = 0; k < Q; ++k) {
                    const float4 v = *reinterpret_cast<const float4*>(src + 4 * k);
                    update[4 * k] += v.x;
                    update[4 * k + 1] += v.y;
                    update[4 * k + 2] += v.z;
                    update[4 * k + 3] += v.w;
                }
            }
        } else {
            for (int part = 0; part < p.parts; ++part, src += p.stride) {
#pragma unroll
                for (int k = 0; k < V; ++k) update[k] += src[k];
            }
        }
#pragma unroll
        for (int k = 0; k < V; ++k) update[k] = Elem<T>::round(update[k]);
    }
    if (V > 1) {
        Vec16<T> a = load_vec16(x + row_offset + i);
#pragma unroll
        for (int k = 0; k < V; ++k) s[k] = (float)a.v[k];
        if (!PARTIAL && d) {
            Vec16<T> b = load_vec16(d + row_offset + i);
#pragma unroll
            for (int k = 0; k < V; ++k) update[k] = (float)b.v[k];
        }
    } else {
        s[0] = (float)x[row_offset + i];
        if (!PARTIAL && d) update[0] = (float)d[row_offset + i];
    }
    if (any) {
#pragma unroll
        for (int k = 0; k < V; ++k) s[k] = Elem<T>::round(s[k] + update[k]);
    }
}

// PARTIAL: the update comes as partial sums (a kernel of its own, so that the plain one keeps its registers).
template <typename T, int V, bool PARTIAL>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(T* __restrict__ resid, const T* __restrict__ delta, PartialSums partial,
                                                          const float* __restrict__ weight, float eps,
                                                          T* __restrict__ out, const int* __restrict__ rows, int width) {
    // The first CACHE vectors of a thread stay in registers between the two passes (a row of up
    // to 256 * V * CACHE elements is read from memory once); what lies beyond is read again.
    constexpr int CACHE = 4;
    __shared__ float scratch[16];
    const int src_row = rows ? rows[blockIdx.x] : blockIdx.x;
    const size_t row_offset = (size_t)src_row * width;
    T* x = resid + row_offset;
    T* y = out + (size_t)blockIdx.x * width;
    const bool updated = PARTIAL || delta;
    const int stride = blockDim.x * V;
    float kept[CACHE][V];
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const int i = threadIdx.x * V + c * stride;
        if (i < width) {
            load_sum<T, V, PARTIAL>(resid, delta, partial, row_offset, i, kept[c]);
#pragma unroll
            for (int k = 0; k < V; ++k) sq += kept[c][k] * kept[c][k];
        }
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride) {
        float s[V];
        load_sum<T, V, PARTIAL>(resid, delta, partial, row_offset, i, s);
#pragma unroll
        for (int k = 0; k < V; ++k) sq += s[k] * s[k];
    }
    const float total = block_sum(sq, scratch);
    const float rstd = rsqrtf(total / (float)width + eps);
    auto emit = [&](int i, const float (&s)[V]) {
        if (V > 1) {
            Vec16<T> o, r;
#pragma unroll
            for (int k = 0; k < V; ++k) {
                r.v[k] = (T)s[k];
                o.v[k] = (T)(s[k] * rstd * weight[i + k]);
            }
            if (updated && !rows) store_vec16(x + i, r);
            store_vec16(y + i, o);
        } else {
            if (updated && !rows) x[i] = (T)s[0];
            y[i] = (T)(s[0] * rstd * weight[i]);
        }
    };
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const int i = threadIdx.x * V + c * stride;
        if (i < width) emit(i, kept[c]);
    }
    for (int i = threadIdx.x * V + CACHE * stride; i < width; i += stride) {
        float s[V];
        load_sum<T, V, PARTIAL>(resid, delta, partial, row_offset, i, s);
        emit(i, s);
    }
}

// ------------------------------------------------------------------------------------------
// SwiGLU: out[t, i] = silu(gu[t, i]) * gu[t, I + i], silu(g) = g * sigmoid(g).
template <typename T, int V>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter) {
    const int t = blockIdx.y;
    const int i = (blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (i >= inter) return;
    const T* g = gate_up + (size_t)t * 2 * inter + i;
    const T* u = g + inter;
    T* o = out + (size_t)t * inter + i;
    if (V > 1) {
        Vec16<T> a = load_vec16(g), b = load_vec16(u), r;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const float gv = (float)a.v[k];
            r.v[k] = (T)(gv / (1.f + expf(-gv)) * (float)b.v[k]);
        }
        store_vec16(o, r);
    } else {
        const float gv = (float)g[0];
        o[0] = (T)(gv / (1.f + expf(-gv)) * (float)u[0]);
    }
}

// ------------------------------------------------------------------------------------------
// y[t, n] += bias[n] (bias float32).
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, int n, size_t total) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) y[i] = (T)((float)y[i] + bias[i % n]);
}

// ------------------------------------------------------------------------------------------
template <typename T>
static int launch_embedding(const void* table, const int* ids, void* out, int n_tokens, int width, int vocab, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const bool vec = width % Elem<T>::kVec == 0;
    if (vec) embedding_kernel<T, true><<<n_tokens, 256, 0, stream>>>((const T*)table, ids, (T*)out, width, vocab);
    else embedding_kernel<T, false><<<n_tokens, 256, 0, stream>>>((const T*)table, ids, (T*)out, width, vocab);
    LSA_LAUNCH_CHECK();
}

template <typename T>
static int launch_add_rmsnorm(void* resid, const void* delta, PartialSums partial, const float* weight, float eps, void* out,
                              const int* rows, int n_out, int width, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (delta && partial.sums) return -1;
#define LSA_ADD_RMSNORM(V, PARTIAL) \
    add_rmsnorm_kernel<T, V, PARTIAL><<<n_out, 256, 0, stream>>>((T*)resid, (const T*)delta, partial, weight, eps, (T*)out, rows, width)
    const bool vectors = width % Elem<T>::kVec == 0;
    if (partial.sums) {
        if (vectors) LSA_ADD_RMSNORM(Elem<T>::kVec, true);
        else LSA_ADD_RMSNORM(1, true);
    } else {
        if (vectors) LSA_ADD_RMSNORM(Elem<T>::kVec, false);
        else LSA_ADD_RMSNORM(1, false);
    }
#undef LSA_ADD_RMSNORM
    LSA_LAUNCH_CHECK();
}

template <typename T>
static int launch_swiglu(const void* gate_up, void* out, int n_tokens, int inter, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (inter % Elem<T>::kVec == 0) {
        constexpr int V = Elem<T>::kVec;
        dim3 grid((inter / V + 255) / 256, n_tokens);
        swiglu_kernel<T, V><<<grid, 256, 0, stream>>>((const T*)gate_up, (T*)out, inter);
    } else {
        dim3 grid((inter + 255) / 256, n_tokens);
        swiglu_kernel<T, 1><<<grid, 256, 0, stream>>>((const T*)gate_up, (T*)out, inter);
    }
    LSA_LAUNCH_CHECK();
}

template <typename T>
static int launch_add_bias(void* y, const float* bias, int n_tokens, int n, hipStream_t stream) {
    const size_t total = (size_t)n_tokens * n;
    if (total == 0) return 0;
    add_bias_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>((T*)y, bias, n, total);
    LSA_LAUNCH_CHECK();
}

// dtype: 0 = float32, 1 = bfloat16
LSA_EXPORT int lsa_embedding(int dtype, const void* table, const int* ids, void* out, int n_tokens, int width, int vocab, hipStream_t stream) {
    return dtype ? launch_embedding<bf16_t>(table, ids, out, n_tokens, width, vocab, stream)
                 : launch_embedding<float>(table, ids, out, n_tokens, width, vocab, stream);
}
LSA_EXPORT int lsa_add_rmsnorm(int dtype, void* resid, const void* delta, const float* weight, float eps, void* out,
                               const int* rows, int n_out, int width, hipStream_t stream) {
    const PartialSums none = {nullptr, 0, 0};
    return dtype ? launch_add_rmsnorm<bf16_t>(resid, delta, none, weight, eps, out, rows, n_out, width, stream)
                 : launch_add_rmsnorm<float>(resid, delta, none, weight, eps, out, rows, n_out, width, stream);
}
// The same with the update given as `parts` partial sums in float32, [parts, rows of resid, width]: they are added
// up and rounded to the stream's type, as a product that had not been split would have been, then added to the stream.
LSA_EXPORT int lsa_add_rmsnorm_partial_sums(int dtype, void* resid, const float* sums, int parts, long part_stride,
                                            const float* weight, float eps, void* out, const int* rows, int n_out, int width,
                                            hipStream_t stream) {
    if (!sums || parts <= 0 || part_stride < 0) return -1;
    const PartialSums partial = {sums, parts, (size_t)part_stride};
    return dtype ? launch_add_rmsnorm<bf16_t>(resid, nullptr, partial, weight, eps, out, rows, n_out, width, stream)
                 : launch_add_rmsnorm<float>(resid, nullptr, partial, weight, eps, out, rows, n_out, width, stream);
}
LSA_EXPORT int lsa_swiglu(int dtype, const void* gate_up, void* out, int n_tokens, int inter, hipStream_t stream) {
    return dtype ? launch_swiglu<bf16_t>(gate_up, out, n_tokens, inter, stream)
                 : launch_swiglu<float>(gate_up, out, n_tokens, inter, stream);
}
LSA_EXPORT int lsa_add_bias(int dtype, void* y, const float* bias, int n_tokens, int n, hipStream_t stream) {
    return dtype ? launch_add_bias<bf16_t>(y, bias, n_tokens, n, stream)
                 : launch_add_bias<float>(y, bias, n_tokens, n, stream);
}

// ------------------------------------------------------------------------------------------
// A plain read of memory, for scale: what the memory system delivers to a kernel that does nothing but read, from a
// given number of workgroups.  Every workgroup streams a contiguous share of `bytes` with 16-byte loads, eight of
// them in flight per lane, and adds what it reads up (the sum is written only if it has a value it cannot have, so
// that the loads stay).  The rooflines of the step's kernels are read against this, not only against the data sheet.
typedef float read_f32x4 __attribute__((ext_vector_type(4)));
__global__ void plain_read_kernel(const read_f32x4* __restrict__ data, float* __restrict__ sink, size_t pieces_per_workgroup) {
    const read_f32x4* base = data + (size_t)blockIdx.x * pieces_per_workgroup;
    read_f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    const size_t stride = blockDim.x;
    for (size_t first = threadIdx.x; first < pieces_per_workgroup; first += stride * 8) {
        read_f32x4 piece[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t at = first + u * stride;
            piece[u] = base[at < pieces_per_workgroup ? at : first];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += piece[u];
    }
    if (sum.x + sum.y + sum.z + sum.w == 12345.678f) sink[0] = 1.f;
}
// `bytes` of `data` (a multiple of 16 * workgroups is read; the rest is left out), `threads` per workgroup (64 to 1024).
LSA_EXPORT int lsa_plain_read(const void* data, float* sink, long bytes, int workgroups, int threads, hipStream_t stream) {
    if (!data || !sink || workgroups <= 0 || threads < 64 || threads > 1024 || threads % 64 || bytes < 16L * workgroups) return -1;
    plain_read_kernel<<<workgroups, threads, 0, stream>>>((const read_f32x4*)data, sink, (size_t)(bytes / 16 / workgroups));
    LSA_LAUNCH_CHECK();
}
