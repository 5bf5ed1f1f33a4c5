// Per-sample inertia, euclidean distances and empty-cluster relocation for gfx950.
// All three are HBM-bound passes over X_t: one thread per sample, features read with
// coalesced loads (consecutive lanes = consecutive samples of one feature row).
#include "kmx_common.h"

#include <type_traits>

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
// SUM: nothing is written per sample; the workgroup's total goes to its slot of `partial` in fp64
// (fixed order inside the workgroup, so the result does not depend on timing).  With few samples
// of many features the launch has a second grid dimension and workgroup (x, y) takes the y-th
// stretch of the features only: a thread that walks hundreds of feature rows alone, with a few
// hundred threads on the whole device, is a chain of trips to memory.
template <typename T, bool LDS_CENTROIDS, bool SUM>
__global__ __launch_bounds__(256) void per_sample_inertia_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight,
    const T* __restrict__ centroids_t, const uint32_t* __restrict__ labels, T* __restrict__ out,
    double* __restrict__ partial, int64_t n, int d, int k, int vec_ok) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* cs = reinterpret_cast<T*>(smem_raw);  // the workgroup's feature rows of centroids_t, same layout
    const int f_chunk = (d + (int)gridDim.y - 1) / (int)gridDim.y;
    const int f_begin = (int)blockIdx.y * f_chunk;
    const int f_end = f_begin + f_chunk < d ? f_begin + f_chunk : d;
    if (LDS_CENTROIDS) {
        for (int idx = threadIdx.x; idx < (f_end - f_begin) * k; idx += 256) cs[idx] = centroids_t[(size_t)f_begin * k + idx];
        __syncthreads();
    }
    // (row f of the centroids: cent + f k)
    const T* __restrict__ cent = LDS_CENTROIDS ? cs - (size_t)f_begin * k : centroids_t;
    const int64_t n_groups = (n + 3) >> 2;
    const int64_t stride = (int64_t)gridDim.x * 256;
    double total = 0.0;
    (void)total;
    for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < n_groups; g += stride) {
        const int64_t i0 = g * 4;
        const bool full = vec_ok && (i0 + 4 <= n);
        uint32_t c[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) c[r] = (i0 + r < n) ? labels[i0 + r] : 0u;
        T acc[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll 4
        for (int f = f_begin; f < f_end; ++f) {
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
        if constexpr (SUM) {
            // samples past n have x = 0 and label 0: their value is dropped here
#pragma unroll
            for (int r = 0; r < 4; ++r) total += (i0 + r < n) ? (double)acc[r] : 0.0;
        } else {
            store4<T>(out, i0, n, full, acc);
        }
    }
    if constexpr (SUM) {
        __shared__ double wave_part[4];
        total = kmx_block_sum<double>(total, wave_part);
        if (threadIdx.x == 0) partial[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = total;
    }
}

// out[0] = sum of the workgroup partials, in order.
template <typename T>
__global__ __launch_bounds__(256) void inertia_total_kernel(const double* __restrict__ partial, int count,
                                                            T* __restrict__ out) {
    __shared__ double wave_part[4];
    double v = 0.0;
    for (int i = threadIdx.x; i < count; i += 256) v += partial[i];
    v = kmx_block_sum<double>(v, wave_part);
    if (threadIdx.x == 0) out[0] = (T)v;
}

// Square root of a non-negative squared distance.  fp32: the hardware approximation (1 ulp)
// refined by one Newton step on the residual, which is within an ulp of the correctly rounded
// root at a third of its cost; tiny arguments, where the approximation loses bits, take the
// library routine.
__device__ __forceinline__ float dist_sqrt(float a) {
    if (a < 1e-30f) return sqrtf(a);
    const float s = __builtin_amdgcn_sqrtf(a);
    const float half_inv = 0.5f * __builtin_amdgcn_rcpf(s);
    return fmaf(fmaf(-s, s, a), half_inv, s);
}
__device__ __forceinline__ double dist_sqrt(double a) { return sqrt(a); }

// distances_t[c, i] = sqrt(sum_f (c_fc - x_fi)^2).  Output bound (k values written per
// sample).  A thread keeps the features of four consecutive samples in registers (d <= DREG);
// the workgroup's share of the centroids (blockIdx.y: `c_chunk` of them, a multiple of 4) is
// staged in LDS, and the thread walks it four centroids at a time: one 128-bit broadcast read
// per feature, sixteen independent sums, one 128-bit store per centroid row.
template <typename T, int DREG>
__global__ __launch_bounds__(256) void euclidean_distances_reg_kernel(
    const T* __restrict__ X_t, const T* __restrict__ centroids_t, T* __restrict__ distances_t,
    int64_t n, int d, int k, int vec_ok, int c_chunk) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* cs = reinterpret_cast<T*>(smem_raw);  // [d][c_chunk]
    const int c_begin = blockIdx.y * c_chunk;
    for (int idx = threadIdx.x; idx < d * c_chunk; idx += 256) {
        const int f = idx / c_chunk, c = c_begin + idx % c_chunk;
        cs[idx] = c < k ? centroids_t[(size_t)f * k + c] : T(0);
    }
    __syncthreads();
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
        for (int c4 = 0; c4 < c_chunk; c4 += 4) {
            T acc[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][r] = T(0);
#pragma unroll
            for (int f = 0; f < DREG; ++f) {
                if (f < d) {
                    T cv[4];
                    load4<T>(cs + f * c_chunk, c4, c_chunk, true, cv);  // same address in every lane
#pragma unroll
                    for (int j = 0; j < 4; ++j)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const T diff = cv[j] - x[f][r];
                            acc[j][r] = fma(diff, diff, acc[j][r]);
                        }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = c_begin + c4 + j;
                if (c < k) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[j][r] = dist_sqrt(acc[j][r]);
                    store4<T>(distances_t + (size_t)c * n, i0, n, full, acc[j]);
                }
            }
        }
    }
}

// Any d: a workgroup owns a tile of DT_S samples x DC centroids, a thread a 4 x (DC / 8) block of
// it; the features are staged DT_K at a time through LDS (both arrays are feature-major, as the
// tiles: a stage is a copy of rows, 128-bit loads where alignment allows), the next stage's
// loads in flight during the arithmetic.  Per staged feature a thread reads its four samples
// and its centroids from LDS (the centroid reads are broadcasts) and updates its sums with a
// difference and a fused multiply-add each, features in order: vector-ALU bound.
// DC = 64, or 16 for up to 32 clusters: with 10 clusters a tile of 64 is five sixths padding,
// and the kernel took ten times what reading X takes.
constexpr int DT_S = 128, DT_C = 64, DT_C_FEW = 16, DT_K = 16;

// 128-bit vectors per thread of a staged tile of COLS columns (fewer vectors than threads: the
// first threads take one)
template <typename T, int COLS>
constexpr int dt_vectors() {
    return (DT_K * (COLS / (16 / (int)sizeof(T))) + 255) / 256;
}

template <typename T, int COLS>
__device__ __forceinline__ void dt_stage_load(T (*regs)[16 / sizeof(T)], const T* __restrict__ base, int64_t len,
                                              int64_t c0, int d, int f0, bool vec_ok) {
    constexpr int V = 16 / sizeof(T);                 // elements per 128-bit vector
    constexpr int PER_ROW = COLS / V;                 // vectors per staged row
    constexpr int N = dt_vectors<T, COLS>();          // vectors per thread
#pragma unroll
    for (int l = 0; l < N; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int f = f0 + g / PER_ROW;
        const int64_t c = c0 + (int64_t)V * (g % PER_ROW);
#pragma unroll
        for (int e = 0; e < V; ++e) regs[l][e] = T(0);
        if (f < d && g < DT_K * PER_ROW) {
            const T* __restrict__ src = base + (size_t)f * (size_t)len + c;
            if (vec_ok && c + V <= len) {
                using Vec = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
                union {
                    Vec v;
                    T s[V];
                } u;
                u.v = *reinterpret_cast<const Vec*>(src);
#pragma unroll
                for (int e = 0; e < V; ++e) regs[l][e] = u.s[e];
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e)
                    if (c + e < len) regs[l][e] = src[e];
            }
        }
    }
}

template <typename T, int COLS>
__device__ __forceinline__ void dt_stage_store(T (*tile)[COLS], const T (*regs)[16 / sizeof(T)]) {
    constexpr int V = 16 / sizeof(T);
    constexpr int PER_ROW = COLS / V;
    constexpr int N = dt_vectors<T, COLS>();
#pragma unroll
    for (int l = 0; l < N; ++l) {
        const int g = threadIdx.x + 256 * l;
        if (g < DT_K * PER_ROW) {
#pragma unroll
            for (int e = 0; e < V; ++e) tile[g / PER_ROW][V * (g % PER_ROW) + e] = regs[l][e];
        }
    }
}

template <typename T, int DC>
__global__ __launch_bounds__(256) void euclidean_distances_tiled_kernel(
    const T* __restrict__ X_t, const T* __restrict__ centroids_t, T* __restrict__ distances_t,
    int64_t n, int d, int k, int x_vec, int c_vec, int out_vec) {
    constexpr int V = 16 / sizeof(T);
    constexpr int CT = DC / 8;  // centroids per thread
    __shared__ __align__(16) T xs[DT_K][DT_S];
    __shared__ __align__(16) T cs[DT_K][DC];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int64_t i0 = (int64_t)blockIdx.x * DT_S;
    const int c0 = blockIdx.y * DC;
    T rx[dt_vectors<T, DT_S>()][V], rc[dt_vectors<T, DC>()][V];
    T acc[CT][4];
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[c][i] = T(0);

    dt_stage_load<T, DT_S>(rx, X_t, n, i0, d, 0, x_vec != 0);
    dt_stage_load<T, DC>(rc, centroids_t, k, c0, d, 0, c_vec != 0);
    const int n_stages = (d + DT_K - 1) / DT_K;
    for (int st = 0; st < n_stages; ++st) {
        __syncthreads();  // the previous stage's reads are over
        dt_stage_store<T, DT_S>(xs, rx);
        dt_stage_store<T, DC>(cs, rc);
        __syncthreads();
        if (st + 1 < n_stages) {
            dt_stage_load<T, DT_S>(rx, X_t, n, i0, d, (st + 1) * DT_K, x_vec != 0);
            dt_stage_load<T, DC>(rc, centroids_t, k, c0, d, (st + 1) * DT_K, c_vec != 0);
        }
        // (rows past d hold zeros on both sides: their differences add nothing)
#pragma unroll
        for (int kk = 0; kk < DT_K; ++kk) {
            T xv[4], cv[CT];
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[i] = xs[kk][4 * tx + i];
#pragma unroll
            for (int c = 0; c < CT; ++c) cv[c] = cs[kk][CT * ty + c];
#pragma unroll
            for (int c = 0; c < CT; ++c)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const T diff = cv[c] - xv[i];
                    acc[c][i] = fma(diff, diff, acc[c][i]);
                }
        }
    }
    const int64_t i = i0 + 4 * tx;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const int cc = c0 + CT * ty + c;
        if (cc >= k) continue;
        T* __restrict__ dst = distances_t + (size_t)cc * (size_t)n + i;
        if (sizeof(T) == 4 && out_vec && i + 4 <= n) {
            *reinterpret_cast<float4*>(dst) = make_float4((float)dist_sqrt(acc[c][0]), (float)dist_sqrt(acc[c][1]),
                                                          (float)dist_sqrt(acc[c][2]), (float)dist_sqrt(acc[c][3]));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (i + e < n) dst[e] = dist_sqrt(acc[c][e]);
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

int stream_grid(int64_t n);
// fp64 partial sums a launch of the summing kernel may write: eight per compute unit, or one per
// workgroup of its first grid dimension where that is more
int64_t inertia_partial_slots(int64_t n) {
    const int64_t a = (int64_t)kmx_num_cus() * 8, b = stream_grid(kmx_cdiv(n, 4));
    return a > b ? a : b;
}

int stream_grid(int64_t n) {
    int64_t blocks = kmx_cdiv(n, 256);
    const int64_t cap = (int64_t)kmx_num_cus() * 8;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace

int32_t kmx_inertia_total_launch(const double* partial, int count, void* out, int32_t dtype, hipStream_t stream) {
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((inertia_total_kernel<float>), dim3(1), dim3(256), 0, stream, partial, count, (float*)out);
    else
        hipLaunchKernelGGL((inertia_total_kernel<double>), dim3(1), dim3(256), 0, stream, partial, count, (double*)out);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

extern "C" {

static int32_t inertia_launch(const void* X_t, const void* sample_weight, const void* centroids_t,
                              const uint32_t* labels, void* out, double* partial, int64_t n, int32_t d, int32_t k,
                              int32_t dtype, hipStream_t stream) {
    const bool sum = partial != nullptr;
    const int grid = stream_grid(kmx_cdiv(n, 4));
    const size_t es = kmx_dtype_size(dtype);
    auto al16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    const int vec_ok =
        (n % 4 == 0) && al16(X_t) && (sum || al16(out)) && (sample_weight == nullptr || al16(sample_weight));
    // the sum over few samples of many features: the features split over the second grid dimension
    // until there are about four workgroups per compute unit (and at least 16 features each)
    int gy = 1;
    if (sum) {
        gy = (int)kmx_cdiv((int64_t)kmx_num_cus() * 4, grid);
        if (gy > d / 16) gy = d / 16;
        if ((int64_t)gy * grid > inertia_partial_slots(n)) gy = (int)(inertia_partial_slots(n) / grid);
        if (gy < 1) gy = 1;
    }
    const int f_chunk = (int)kmx_cdiv(d, gy);
    const size_t lds = (size_t)f_chunk * k * es;
    const bool in_lds = lds <= 48 * 1024;
#define KMX_INERTIA(T, L, S)                                                                       \
    hipLaunchKernelGGL((per_sample_inertia_kernel<T, L, S>), dim3(grid, gy), dim3(256), (L) ? lds : 0,  \
                       stream, (const T*)X_t, (const T*)sample_weight, (const T*)centroids_t,      \
                       labels, (S) ? nullptr : (T*)out, partial, n, d, k, vec_ok)
#define KMX_INERTIA_T(T)                                                        \
    do {                                                                        \
        if (in_lds && sum) KMX_INERTIA(T, true, true);                          \
        else if (in_lds) KMX_INERTIA(T, true, false);                           \
        else if (sum) KMX_INERTIA(T, false, true);                              \
        else KMX_INERTIA(T, false, false);                                      \
    } while (0)
    if (dtype == KMX_F32) KMX_INERTIA_T(float); else KMX_INERTIA_T(double);
#undef KMX_INERTIA_T
#undef KMX_INERTIA
    if (sum) {
        if (dtype == KMX_F32)
            hipLaunchKernelGGL((inertia_total_kernel<float>), dim3(1), dim3(256), 0, stream, partial, grid * gy, (float*)out);
        else
            hipLaunchKernelGGL((inertia_total_kernel<double>), dim3(1), dim3(256), 0, stream, partial, grid * gy, (double*)out);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

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
    return inertia_launch(X_t, sample_weight, centroids_t, labels, out, nullptr, n, d, k, dtype, (hipStream_t)stream_);
}

size_t kmx_inertia_workspace_bytes(int64_t n) {
    if (n <= 0) return 0;
    return kmx_align256((size_t)inertia_partial_slots(n) * sizeof(double));
}

int32_t kmx_inertia(const void* X_t, const void* sample_weight, const void* centroids_t, const uint32_t* labels,
                    void* out_total, void* workspace, size_t workspace_bytes, int64_t n, int32_t d, int32_t k,
                    int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(out_total);
    KMX_REQUIRE_PTR(workspace);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (workspace_bytes < kmx_inertia_workspace_bytes(n)) return KMX_ERR_WORKSPACE;
    return inertia_launch(X_t, sample_weight, centroids_t, labels, out_total, (double*)workspace, n, d, k, dtype,
                          (hipStream_t)stream_);
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
    // register kernel: the centroid range is split over blockIdx.y until there are about six
    // workgroups per compute unit (a thread's walk over the centroids is one dependent chain)
    const int64_t wgx = stream_grid(kmx_cdiv(n, 4));
    int64_t gy = kmx_cdiv((int64_t)kmx_num_cus() * 6, wgx);
    if (gy > kmx_cdiv(k, 16)) gy = kmx_cdiv(k, 16);
    if (gy < 1) gy = 1;
    const int c_chunk = (int)(4 * kmx_cdiv(kmx_cdiv(k, gy), 4));
    gy = kmx_cdiv(k, c_chunk);
    const size_t es = kmx_dtype_size(dtype);
    const size_t lds = (size_t)d * c_chunk * es;
    const dim3 rgrid((unsigned)wgx, (unsigned)gy);
    if (dtype == KMX_F32 && d <= 32 && lds <= 64 * 1024) {
        if (d <= 16)
            hipLaunchKernelGGL((euclidean_distances_reg_kernel<float, 16>), rgrid, dim3(256), lds, stream,
                               (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d, k, vec_ok,
                               c_chunk);
        else
            hipLaunchKernelGGL((euclidean_distances_reg_kernel<float, 32>), rgrid, dim3(256), lds, stream,
                               (const float*)X_t, (const float*)centroids_t, (float*)distances_t, n, d, k, vec_ok,
                               c_chunk);
    } else if (dtype == KMX_F64 && d <= 16 && lds <= 64 * 1024) {
        hipLaunchKernelGGL((euclidean_distances_reg_kernel<double, 16>), rgrid, dim3(256), lds, stream,
                           (const double*)X_t, (const double*)centroids_t, (double*)distances_t, n, d, k, vec_ok,
                           c_chunk);
    } else {
        const int dc = k <= 2 * DT_C_FEW ? DT_C_FEW : DT_C;
        const dim3 tgrid((unsigned)kmx_cdiv(n, DT_S), (unsigned)kmx_cdiv(k, dc));
        const int per_vec = (int)(16 / es);
        const int x_vec = (n % per_vec == 0) && al16(X_t), c_vec = (k % per_vec == 0) && al16(centroids_t);
#define KMX_DIST_TILED(T, DC, OUT_VEC)                                                                 \
    hipLaunchKernelGGL((euclidean_distances_tiled_kernel<T, DC>), tgrid, dim3(256), 0, stream,         \
                       (const T*)X_t, (const T*)centroids_t, (T*)distances_t, n, d, k, x_vec, c_vec, OUT_VEC)
        if (dtype == KMX_F32) {
            if (dc == DT_C_FEW) KMX_DIST_TILED(float, DT_C_FEW, vec_ok); else KMX_DIST_TILED(float, DT_C, vec_ok);
        } else {
            if (dc == DT_C_FEW) KMX_DIST_TILED(double, DT_C_FEW, 0); else KMX_DIST_TILED(double, DT_C, 0);
        }
#undef KMX_DIST_TILED
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
