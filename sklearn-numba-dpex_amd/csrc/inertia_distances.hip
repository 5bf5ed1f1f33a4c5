// Per-sample inertia, euclidean distances and empty-cluster relocation for gfx950.
// All three are HBM-bound passes over X_t: one thread per sample, features read with
// coalesced loads (consecutive lanes = consecutive samples of one feature row).
#include "kmx_common.h"

namespace {

// out[i] = w_i * sum_f (x_fi - c_f,label_i)^2, features accumulated in order.
template <typename T>
__global__ __launch_bounds__(256) void per_sample_inertia_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight,
    const T* __restrict__ centroids_t, const uint32_t* __restrict__ labels, T* __restrict__ out,
    int64_t n, int d, int k) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const uint32_t c = labels[i];
        T acc = T(0);
#pragma unroll 4
        for (int f = 0; f < d; ++f) {
            const T diff = X_t[(size_t)f * n + i] - centroids_t[(size_t)f * k + c];
            acc += diff * diff;
        }
        out[i] = sample_weight ? acc * sample_weight[i] : acc;
    }
}

// distances_t[c, i] = sqrt(sum_f (c_fc - x_fi)^2).  The thread keeps KC running sums for a
// window of centroids (wave-uniform centroid loads) and writes KC coalesced rows.
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
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(out);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const int grid = stream_grid(n);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((per_sample_inertia_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (const float*)X_t, (const float*)sample_weight,
                           (const float*)centroids_t, labels, (float*)out, n, d, k);
    else
        hipLaunchKernelGGL((per_sample_inertia_kernel<double>), dim3(grid), dim3(256), 0, stream,
                           (const double*)X_t, (const double*)sample_weight,
                           (const double*)centroids_t, labels, (double*)out, n, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_euclidean_distances(const void* X_t, const void* centroids_t, void* distances_t,
                                int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream_) {
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(distances_t);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const int grid = stream_grid(n);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((euclidean_distances_kernel<float, 8>), dim3(grid), dim3(256), 0, stream,
                           (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d,
                           k);
    else
        hipLaunchKernelGGL((euclidean_distances_kernel<double, 8>), dim3(grid), dim3(256), 0,
                           stream, (const double*)X_t, (const double*)centroids_t,
                           (double*)distances_t, n, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_relocate_empty_clusters(const void* X_t, const void* sample_weight,
                                    const uint32_t* labels, const int64_t* far_samples,
                                    const uint32_t* empty_clusters, int32_t n_relocated,
                                    void* per_sample_inertia, void* sums_t, void* cluster_sizes,
                                    int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream_) {
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
