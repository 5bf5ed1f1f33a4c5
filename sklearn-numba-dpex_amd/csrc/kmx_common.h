// Shared helpers for the gfx950 KMeans kernels: argument checks, dtype dispatch,
// wave64/block reductions.  Internal to the library; the public ABI is
// include/mi355x_kmeans.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi355x_kmeans.h"

#define KMX_WAVE 64

#define KMX_REQUIRE_PTR(p) \
    do {                   \
        if ((p) == nullptr) return KMX_ERR_NULL_POINTER; \
    } while (0)

#define KMX_REQUIRE_DTYPE(dt) \
    do {                      \
        if ((dt) != KMX_F32 && (dt) != KMX_F64) return KMX_ERR_BAD_DTYPE; \
    } while (0)

// First statement of every entry point that launches kernels: hipGetLastError reports the
// last error of ANY earlier runtime call of the thread (another library's probe included), so
// a stale one is dropped here and KMX_LAUNCH_CHECK only sees this library's own launches.
#define KMX_ENTRY() (void)hipGetLastError()

#define KMX_LAUNCH_CHECK()                    \
    do {                                      \
        hipError_t e_ = hipGetLastError();    \
        if (e_ != hipSuccess) return (int32_t)e_; \
    } while (0)

static inline size_t kmx_align256(size_t x) { return (x + 255) & ~(size_t)255; }
static inline size_t kmx_dtype_size(int32_t dtype) { return dtype == KMX_F64 ? 8 : 4; }
static inline int64_t kmx_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Number of compute units of the current device (cached); 256 on MI355X.
int32_t kmx_num_cus();

// ---------------------------------------------------------------------------- device side

template <typename T>
__device__ __forceinline__ T kmx_inf();
template <>
__device__ __forceinline__ float kmx_inf<float>() { return __builtin_huge_valf(); }
template <>
__device__ __forceinline__ double kmx_inf<double>() { return __builtin_huge_val(); }

// Sum over the 64 lanes of a wave; every lane receives the total.
template <typename T>
__device__ __forceinline__ T kmx_wave_sum(T v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, KMX_WAVE);
    return v;
}

// Sum over a block of up to 1024 threads; result valid in thread 0.  `scratch` holds
// at least blockDim.x / 64 elements of T in LDS.  Fixed order, hence reproducible.
template <typename T>
__device__ __forceinline__ T kmx_block_sum(T v, T* scratch) {
    v = kmx_wave_sum(v);
    const int lane = threadIdx.x & (KMX_WAVE - 1);
    const int wave = threadIdx.x / KMX_WAVE;
    const int n_waves = (blockDim.x + KMX_WAVE - 1) / KMX_WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    T total = T(0);
    if (threadIdx.x == 0) {
        for (int i = 0; i < n_waves; ++i) total += scratch[i];
    }
    return total;
}

// Hardware floating-point atomic add (LDS or global), result unused.
template <typename T>
__device__ __forceinline__ void kmx_atomic_add(T* addr, T v) {
    unsafeAtomicAdd(addr, v);
}

// (value, index) minimum with the lowest index winning ties.
template <typename T>
__device__ __forceinline__ void kmx_argmin_combine(T& v, int64_t& i, T ov, int64_t oi) {
    if (ov < v || (ov == v && oi < i)) {
        v = ov;
        i = oi;
    }
}
