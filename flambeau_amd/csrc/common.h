// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wave64 reductions, the paged-cache address rule and host-side error reporting.
#pragma once
#include <utility>
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define FL_WAVE 64

// dtype codes of the C interface
#define FL_F32 0
#define FL_BF16 1

// f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}): a loop whose index
// is a constant in every turn.
template <int N, typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl<N>(f, std::make_integer_sequence<int, N>{});
}

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, FL_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, FL_WAVE));
    return v;
}

// Sum over a block of NW waves; every thread gets the total.  `lds` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* lds) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) lds[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) t += lds[w];
    return t;
}

// Paged cache of one layer: [n_pages][2 (K,V)][n_kv_heads][page_size * head_dim].
// Token t of a request lives in page table[t / page_size] at row r = t % page_size.
// Within a (page, head) block keys are stored row by row, K[r][d] at r * head_dim + d,
// and values transposed, V[r][d] at d * page_size + r: matrix-core operands want the index
// that is summed over (head dims for Q.K, keys for P.V) contiguous in memory.
struct PagedCache {
    void* base;        // this layer's pool
    int n_kv_heads;
    int page_size;
    int head_dim;
    int n_pages;
};

__device__ __forceinline__ size_t cache_block_offset(const PagedCache& c, int page, int is_v, int kv_head) {
    return (((size_t)page * 2 + is_v) * c.n_kv_heads + kv_head) * (size_t)c.page_size * c.head_dim;
}
__device__ __forceinline__ size_t cache_k_offset(const PagedCache& c, int page, int kv_head, int row, int d) {
    return cache_block_offset(c, page, 0, kv_head) + (size_t)row * c.head_dim + d;
}
__device__ __forceinline__ size_t cache_v_offset(const PagedCache& c, int page, int kv_head, int row, int d) {
    return cache_block_offset(c, page, 1, kv_head) + (size_t)d * c.page_size + row;
}

// ---- host side -----------------------------------------------------------
void fl_set_error(const char* fmt, ...);
int fl_units(void);              // compute units of the current device (runtime.hip)

#define FL_CHECK(cond, ...)                \
    do {                                   \
        if (!(cond)) {                     \
            fl_set_error(__VA_ARGS__);     \
            return -1;                     \
        }                                  \
    } while (0)

#define FL_LAUNCH_CHECK()                                                    \
    do {                                                                     \
        hipError_t e_ = hipGetLastError();                                   \
        if (e_ != hipSuccess) {                                              \
            fl_set_error("%s:%d launch failed: %s", __FILE__, __LINE__,      \
                         hipGetErrorString(e_));                             \
            return -2;                                                       \
        }                                                                    \
    } while (0)

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
