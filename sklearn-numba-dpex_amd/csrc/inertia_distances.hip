// Per-sample inertia, euclidean distances and empty-cluster relocation for gfx950.
// All three are HBM-bound passes over X_t: one thread per sample, features read with
// coalesced loads (consecutive lanes = consecutive samples of one feature row).
#include "kmx_common.h"

namespace {

// Four consecutive values of a row at i0 (128-bit accesses when `full`), zero past n.
template <typename T>
__device__ __forceinline__ void load4(const T* __restrict__ row, int64_t i0, int64_t n, bool full, T (&v)[4]) {
    if (full) {
        if constexpr (sizeof(T) == 4) {
            const float4 q = *reinterpret_cast<const float4*>(row + i0);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
            const double2 a = *reinterpret_cast<const double2*>(row + i0);
            const double2 b = *reinterpret_cast<const double2*>(row + i0 + 2);
            v[0] = a.x; v[1] = a.y; v[2] = b.x; v[3] = b.y;
        }
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (i0 + r < n) ? row[i0 + r] : T(0);
    }
}

template <typename T>
__device__ __forceinline__ void store4(T* __restrict__ row, int64_t i0, int64_t n, bool full, const T (&v)[4]) {
    if (full) {
        if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<float4*>(row + i0) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            *reinterpret_cast<double2*>(row + i0) = make_double2(v[0], v[1]);
            *reinterpret_cast<double2*>(row + i0 + 2) = make_double2(v[2], v[3]);
        }
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (i0 + r < n) row[i0 + r] = v[r];
    }
}

// out[i] = w_i * sum_f (x_fi - c_f,label_i)^2, features accumulated in order.  A thread takes
// four consecutive samples (128-bit loads of every feature row); the centroids are staged in
// LDS when they fit (LDS_CENTROIDS), so that the per-sample gather of the label's centroid
// does not go through the vector memory pipe.
template <typename T, bool LDS_CENTROIDS>
__global__ __launch_bounds__(256) void per_sample_inertia_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight,
    const T* __restrict__ centroids_t, const uint32_t* __restrict__ labels, T* __restrict__ out,
    int64_t n, int d, int k, int vec_ok) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* cs = reinterpret_cast<T*>(smem_raw);  // [d * k], same layout as centroids_t
    if (LDS_CENTROIDS) {
        for (int idx = threadIdx.x; idx < d * k; idx += 256) cs[idx] = centroids_t[idx];
        __syncthreads();
    }
    const T* __restrict__ cent = LDS_CENTROIDS ? cs : centroids_t;
    const int64_t n_groups = (n + 3) >> 2;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < n_groups; g += stride) {
        const int64_t i0 = g * 4;
        const bool full = vec_ok && (i0 + 4 <= n);
        uint32_t c[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) c[r] = (i0 + r < n) ? labels[i0 + r] : 0u;
        T acc[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll 2
        for (int f = 0; f < d; ++f) {
            T x[4];
            load4<T>(X_t + (size_t)f * n, i0, n, full, x);
            const T* __restrict__ crow = cent + (size_t)f * k;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const T diff = x[r] - crow[c[r]];
                acc[r] += diff * diff;
            }
        }
        if (sample_weight) {
            T w[4];
            load4<T>(sample_weight, i0, n, full, w);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] *= w[r];
        }
        store4<T>(out, i0, n, full, acc);
    }
}

// distances_t[c, i] = sqrt(sum_f (c_fc - x_fi)^2).  Output bound (k values written per
// sample).  A thread keeps the features of four consecutive samples in registers (d <= DREG)
// and walks the centroids through wave-uniform loads, writing one 128-bit store per centroid.
template <typename T, int DREG>
__global__ __launch_bounds__(256) void euclidean_distances_reg_kernel(
    const T* __restrict__ X_t, const T* __restrict__ centroids_t, T* __restrict__ distances_t,
    int64_t n, int d, int k, int vec_ok) {
    const int64_t n_groups = (n + 3) >> 2;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < n_groups; g += stride) {
        const int64_t i0 = g * 4;
        const bool full = vec_ok && (i0 + 4 <= n);
        T x[DREG][4];
#pragma unroll
        for (int f = 0; f < DREG; ++f) {
            if (f < d) {
                load4<T>(X_t + (size_t)f * n, i0, n, full, x[f]);
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) x[f][r] = T(0);
            }
        }
        for (int c = 0; c < k; ++c) {
            T acc[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int f = 0; f < DREG; ++f) {
                if (f < d) {
                    const T cv = centroids_t[(size_t)f * k + c];  // wave-uniform
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const T diff = cv - x[f][r];
                        acc[r] = fma(diff, diff, acc[r]);
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = sqrt(acc[r]);
            store4<T>(distances_t + (size_t)c * n, i0, n, full, acc);
        }
    }
}

// Any d: the thread keeps KC running sums for a window of centroids (wave-uniform centroid
// loads) and writes KC coalesced rows; X is re-read per window through the caches.
template <typename T, int KC>
__global__ __launch_bounds__(256) void euclidean_distances_kernel(
    const T* __restrict__ X_t, const T* __restrict__ centroids_t, T* __restrict__ distances_t,
    int64_t n, int d, int k) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        for (int c0 = 0; c0 < k; c0 += KC) {
            T acc[KC];
#pragma unroll
            for (int j = 0; j < KC; ++j) acc[j] = T(0);
            for (int f = 0; f < d; ++f) {
                const T xv = X_t[(size_t)f * n + i];
                const T* __restrict__ crow = centroids_t + (size_t)f * k;
#pragma unroll
                for (int j = 0; j < KC; ++j) {
                    const int c = (c0 + j < k) ? c0 + j : k - 1;
                    const T diff = crow[c] - xv;
                    acc[j] = fma(diff, diff, acc[j]);
                }
            }
#pragma unroll
            for (int j = 0; j < KC; ++j)
                if (c0 + j < k) distances_t[(size_t)(c0 + j) * n + i] = sqrt(acc[j]);
        }
    }
}

// One workgroup per relocated cluster, threads over features.  Several relocations may take
// samples from the same old cluster, hence the atomic subtraction.
template <typename T>
__global__ __launch_bounds__(256) void relocate_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight,
    const uint32_t* __restrict__ labels, const int64_t* __restrict__ far_samples,
    const uint32_t* __restrict__ empty_clusters, T* __restrict__ per_sample_inertia,
    T* __restrict__ sums_t, T* __restrict__ sizes, int64_t n, int d, int k) {
    const int r = blockIdx.x;
    const uint32_t cluster = empty_clusters[r];
    const int64_t sample = far_samples[r];
    const uint32_t old = labels[sample];
    const T w = sample_weight[sample];
    for (int f = threadIdx.x; f < d; f += 256) {
        const T addend = X_t[(size_t)f * n + sample] * w;
        kmx_atomic_add(sums_t + (size_t)f * k + old, -addend);
        sums_t[(size_t)f * k + cluster] = addend;
    }
    if (threadIdx.x == 0) {
        if (per_sample_inertia) per_sample_inertia[sample] = T(0);
        kmx_atomic_add(sizes + old, -w);
        sizes[cluster] = w;
    }
}

int stream_grid(int64_t n) {
    int64_t blocks = kmx_cdiv(n, 256);
    const int64_t cap = (int64_t)kmx_num_cus() * 8;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace

extern "C" {

int32_t kmx_per_sample_inertia(const void* X_t, const void* sample_weight, const void* centroids_t,
                               const uint32_t* labels, void* out, int64_t n, int32_t d, int32_t k,
                               int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(out);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const int grid = stream_grid(kmx_cdiv(n, 4));
    const size_t es = kmx_dtype_size(dtype);
    auto al16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    const int vec_ok = (n % 4 == 0) && al16(X_t) && al16(out) && (sample_weight == nullptr || al16(sample_weight));
    const size_t lds = (size_t)d * k * es;
    const bool in_lds = lds <= 48 * 1024;
#define KMX_INERTIA(T, L)                                                                         \
    hipLaunchKernelGGL((per_sample_inertia_kernel<T, L>), dim3(grid), dim3(256), (L) ? lds : 0,     \
                       stream, (const T*)X_t, (const T*)sample_weight, (const T*)centroids_t,      \
                       labels, (T*)out, n, d, k, vec_ok)
    if (dtype == KMX_F32) {
        if (in_lds) KMX_INERTIA(float, true); else KMX_INERTIA(float, false);
    } else {
        if (in_lds) KMX_INERTIA(double, true); else KMX_INERTIA(double, false);
    }
#undef KMX_INERTIA
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_euclidean_distances(const void* X_t, const void* centroids_t, void* distances_t,
                                int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(distances_t);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    auto al16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    const int vec_ok = (n % 4 == 0) && al16(X_t) && al16(distances_t);
    if (dtype == KMX_F32 && d <= 32) {
        const int grid = stream_grid(kmx_cdiv(n, 4));
        if (d <= 16)
            hipLaunchKernelGGL((euclidean_distances_reg_kernel<float, 16>), dim3(grid), dim3(256), 0, stream,
                               (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d, k, vec_ok);
        else
            hipLaunchKernelGGL((euclidean_distances_reg_kernel<float, 32>), dim3(grid), dim3(256), 0, stream,
                               (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d, k, vec_ok);
    } else if (dtype == KMX_F64 && d <= 16) {
        const int grid = stream_grid(kmx_cdiv(n, 4));
        hipLaunchKernelGGL((euclidean_distances_reg_kernel<double, 16>), dim3(grid), dim3(256), 0, stream,
                           (const double*)X_t, (const double*)centroids_t, (double*)distances_t, n, d, k, vec_ok);
    } else if (dtype == KMX_F32) {
        hipLaunchKernelGGL((euclidean_distances_kernel<float, 8>), dim3(stream_grid(n)), dim3(256), 0, stream,
                           (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d,
                           k);
    } else {
        hipLaunchKernelGGL((euclidean_distances_kernel<double, 8>), dim3(stream_grid(n)), dim3(256), 0,
                           stream, (const double*)X_t, (const double*)centroids_t,
                           (double*)distances_t, n, d, k);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_relocate_empty_clusters(const void* X_t, const void* sample_weight,
                                    const uint32_t* labels, const int64_t* far_samples,
                                    const uint32_t* empty_clusters, int32_t n_relocated,
                                    void* per_sample_inertia, void* sums_t, void* cluster_sizes,
                                    int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(sample_weight);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(far_samples);
    KMX_REQUIRE_PTR(empty_clusters);
    KMX_REQUIRE_PTR(sums_t);
    KMX_REQUIRE_PTR(cluster_sizes);
    if (n <= 0 || d <= 0 || k <= 0 || n_relocated < 0 || n_relocated > k) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (n_relocated == 0) return KMX_OK;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((relocate_kernel<float>), dim3(n_relocated), dim3(256), 0, stream,
                           (const float*)X_t, (const float*)sample_weight, labels, far_samples,
                           empty_clusters, (float*)per_sample_inertia, (float*)sums_t,
                           (float*)cluster_sizes, n, d, k);
    else
        hipLaunchKernelGGL((relocate_kernel<double>), dim3(n_relocated), dim3(256), 0, stream,
                           (const double*)X_t, (const double*)sample_weight, labels, far_samples,
                           empty_clusters, (double*)per_sample_inertia, (double*)sums_t,
                           (double*)cluster_sizes, n, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

}  // extern "C"
