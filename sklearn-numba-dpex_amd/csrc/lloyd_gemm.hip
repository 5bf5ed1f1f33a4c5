// Labels for any shape on the matrix cores (gfx950): a tiled product of the samples with the
// centroids whose epilogue keeps, per sample, the best score and its centroid.
//
// Replaces, for shapes no specialised kernel takes (fp32 beyond 256 features, fp64 beyond 64
// features or with centroids beyond LDS, few clusters of wide samples), the label half of
// fused_lloyd_single_step (sklearn_numba_dpex/kmeans/kernels/lloyd_single_step.py:35-424) and
// assignment (kmeans/kernels/compute_labels.py:29-288): the reference slides windows of
// centroids through local memory and multiplies on the vector ALU; here the products run on
// v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64.  The sums of the update step come from the
// bucketed accumulation (lloyd_bucket.hip).
//
//   * score(i, c) = <x_i, c> - 0.5 ||c||^2, the label is its arg-max with the lowest centroid
//     winning a tie (the reference minimises 0.5 ||c||^2 - <x, c> with a strict comparison in
//     increasing centroid order).
//   * A workgroup of four waves owns 128 samples and walks the centroids in tiles of 128 (one
//     tile of 32 or 64 for that few clusters); the
//     features are staged 16 (fp32) or 8 (fp64) at a time through double-buffered LDS tiles.
//     Both arrays are feature-major in memory, as the tiles are in LDS: a stage is a copy of
//     rows (128-bit loads where alignment allows), rows padded so that the operand reads of a
//     wave fall on distinct banks.  The next stage's loads are in flight during the MFMAs.
//   * A wave multiplies all 128 centroids of the tile with its own 32 samples: centroids are
//     the rows of the MFMA result and samples its columns, so a lane holds scores of ONE
//     sample (fp32) or two (fp64) and the running arg-max needs no exchange until the end,
//     where the two (fp32) or four (fp64) lanes that share a sample are combined.
//   * Accumulators start at -0.5 ||c||^2 (-inf past the last centroid).
#include "lloyd_layout.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v4d __attribute__((ext_vector_type(4)));

constexpr int GT = 128;       // samples per workgroup, centroids per tile
constexpr int GK32 = 16;      // features per stage, fp32
constexpr int GK64 = 8;       // features per stage, fp64
constexpr int GLD32 = GT + 32;  // LDS row length in floats: the two K rows of a wave's read 32 banks apart
constexpr int GLD64 = GT + 16;  // in doubles: the K rows of a half-wave's read 32 banks apart

// One stage of one operand: rows f0 .. f0 + 8 L - 1 of a feature-major array with `len`
// columns, columns c0 .. c0 + 4 GROUPS - 1, zero outside the array.  Thread t takes the groups
// of four columns t, t + 256, ... (row g / GROUPS, columns 4 (g % GROUPS)); GROUPS = 32 (128
// columns: the samples, or a tile of 128 centroids) makes a load cover 8 rows, a tile of 32 or
// 64 centroids 32 or 16.
template <int L, int GROUPS = 32>
__device__ __forceinline__ void stage_load_f32(float4 (&r)[L], const float* __restrict__ base, int64_t len,
                                               int64_t c0, int d, int f0, bool vec_ok) {
#pragma unroll
    for (int l = 0; l < L; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int f = f0 + g / GROUPS;
        const int64_t c = c0 + 4 * (g % GROUPS);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (f < d) {
            const float* __restrict__ src = base + (size_t)f * (size_t)len + c;
            if (vec_ok && c + 4 <= len) {
                v = *reinterpret_cast<const float4*>(src);
            } else {
                if (c + 0 < len) v.x = src[0];
                if (c + 1 < len) v.y = src[1];
                if (c + 2 < len) v.z = src[2];
                if (c + 3 < len) v.w = src[3];
            }
        }
        r[l] = v;
    }
}

template <int L, int LD, int GROUPS = 32>
__device__ __forceinline__ void stage_store_f32(float (*tile)[LD], const float4 (&r)[L]) {
#pragma unroll
    for (int l = 0; l < L; ++l) {
        const int g = threadIdx.x + 256 * l;
        *reinterpret_cast<float4*>(&tile[g / GROUPS][4 * (g % GROUPS)]) = r[l];
    }
}

// The same stage for LISTED samples: column c of the tile is sample cols[.] of X_t (gathered,
// one load per value); a negative index is a column past the end of the list.  (A thread's
// groups of columns are the same in all its rows.)
template <int L>
__device__ __forceinline__ void stage_load_listed_f32(float4 (&r)[L], const float* __restrict__ X_t, int64_t n,
                                                      const int (&cols)[4], int d, int f0) {
#pragma unroll
    for (int l = 0; l < L; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int f = f0 + (g >> 5);
        const bool row_ok = f < d;
        const float* __restrict__ row = X_t + (size_t)(row_ok ? f : 0) * (size_t)n;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool ok = row_ok && cols[e] >= 0;
            const float x = row[ok ? cols[e] : 0];
            v[e] = ok ? x : 0.0f;
        }
        r[l] = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// NA: 32-centroid row tiles per pass over the features (4: tiles of 128 centroids; 1 or 2 for
// up to 32 / 64 clusters, where wider tiles would multiply padding).  A stage copies the 32 NA
// centroid columns in use.  With one row tile a stage is 32 features instead of 16: the small
// centroid tile leaves the LDS for it, and a workgroup has twice the bytes on their way from
// memory (with few clusters the kernel does little arithmetic per byte and waits for X).
// LISTED: the samples are list[0 .. *list_count) instead of 0 .. n (what a screened label
// kernel could not certify); a workgroup without a tile of the list leaves at once.
template <int NA, bool LISTED = false>
__global__ __launch_bounds__(256, 2) void lloyd_gemm_labels_f32_kernel(
    const float* __restrict__ X_t, const float* __restrict__ centroids_t,
    const float* __restrict__ half_norms, uint32_t* __restrict__ labels,
    const kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k, int x_vec, int c_vec,
    const int* __restrict__ list = nullptr, const unsigned int* __restrict__ list_count = nullptr) {
    if (status != nullptr && status->state != KMX_RUNNING) return;
    const int64_t n_work = LISTED ? (int64_t)*list_count : n;
    constexpr int GK = NA == 1 ? 2 * GK32 : GK32;           // features per stage
    constexpr int XL = GK / 8;                              // 128-bit loads per thread and stage, samples
    constexpr int CG = 8 * NA;                              // groups of four columns per centroid row
    constexpr int CL = GK * CG / 256;                       // loads per thread and stage, centroids
    constexpr int CLD = 32 * NA + (NA % 2 == 0 ? 32 : 0);   // row length: = 32 mod 64, as GLD32
    static_assert(GK * CG % 256 == 0 && CLD % 64 == 32, "whole loads per thread; K rows 32 banks apart");
    __shared__ __align__(16) float xs[2][GK][GLD32];
    __shared__ __align__(16) float cs[2][GK][CLD];
    __shared__ float hn[GT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int n_stages = (d + GK - 1) / GK;
    const int64_t n_tiles = (n_work + GT - 1) / GT;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * GT;
        float best = -kmx_inf<float>();
        int bidx = 0;
        int cols[4];  // LISTED: the samples behind the thread's columns of a stage
        if constexpr (LISTED) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t slot = i0 + 4 * (threadIdx.x & 31) + e;
                cols[e] = slot < n_work ? list[slot] : -1;
            }
        }
        auto load_x = [&](float4(&r)[XL], const int f0) {
            if constexpr (LISTED) stage_load_listed_f32<XL>(r, X_t, n, cols, d, f0);
            else stage_load_f32<XL>(r, X_t, n, i0, d, f0, x_vec != 0);
        };
        auto load_c = [&](float4(&r)[CL], const int c0, const int f0) {
            stage_load_f32<CL, CG>(r, centroids_t, k, c0, d, f0, c_vec != 0);
        };
        for (int c0 = 0; c0 < k; c0 += 32 * NA) {
            __syncthreads();  // the previous tile's reads of hn and of the stage buffers are over
            if (threadIdx.x < GT)
                hn[threadIdx.x] = c0 + (int)threadIdx.x < k ? -half_norms[c0 + threadIdx.x] : -kmx_inf<float>();
            float4 rx[XL], rc[CL];
            load_x(rx, 0);
            load_c(rc, c0, 0);
            stage_store_f32<XL, GLD32>(xs[0], rx);
            stage_store_f32<CL, CLD, CG>(cs[0], rc);
            __syncthreads();

            // accumulator register r of lane (j, h): centroid 32 a + 8 (r / 4) + 4 h + r % 4
            v16f acc[NA];
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[a][r] = hn[32 * a + 8 * (r >> 2) + 4 * h + (r & 3)];

            for (int st = 0; st < n_stages; ++st) {
                const int cur = st & 1;
                if (st + 1 < n_stages) {
                    load_x(rx, (st + 1) * GK);
                    load_c(rc, c0, (st + 1) * GK);
                }
#pragma unroll
                for (int s = 0; s < GK / 2; ++s) {
                    // lane (j, h) supplies feature 2 s + h of centroid / sample j of the 32
                    const float bf = xs[cur][2 * s + h][32 * wave + j];
                    float af[NA];
#pragma unroll
                    for (int a = 0; a < NA; ++a) af[a] = cs[cur][2 * s + h][32 * a + j];
#pragma unroll
                    for (int a = 0; a < NA; ++a)
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[a], bf, acc[a], 0, 0, 0);
                }
                if (st + 1 < n_stages) {
                    stage_store_f32<XL, GLD32>(xs[cur ^ 1], rx);
                    stage_store_f32<CL, CLD, CG>(cs[cur ^ 1], rc);
                }
                __syncthreads();
            }

            // increasing centroid order per lane, strict comparison: the lowest index keeps a tie
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float v = acc[a][r];
                    const int c = c0 + 32 * a + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (v > best) {
                        best = v;
                        bidx = c;
                    }
                }
        }
        // the two lanes of a sample
        const float ob = __shfl_xor(best, 32, 64);
        const int oi = __shfl_xor(bidx, 32, 64);
        if (ob > best || (ob == best && oi < bidx)) bidx = oi;
        const int64_t slot = i0 + 32 * wave + j;
        if (h == 0 && slot < n_work) labels[LISTED ? (int64_t)list[slot] : slot] = (uint32_t)bidx;
    }
}

// fp64: thread t takes the pairs of columns t, t + 256, ... (row g / GROUPS, columns
// 2 (g % GROUPS)); GROUPS = 64 for 128 columns, 16 or 32 for a tile of 32 or 64 centroids.
template <int L, int GROUPS = 64>
__device__ __forceinline__ void stage_load_f64(double2 (&r)[L], const double* __restrict__ base, int64_t len,
                                               int64_t c0, int d, int f0, bool vec_ok) {
#pragma unroll
    for (int l = 0; l < L; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int f = f0 + g / GROUPS;
        const int64_t c = c0 + 2 * (g % GROUPS);
        double2 v = make_double2(0.0, 0.0);
        if (f < d) {
            const double* __restrict__ src = base + (size_t)f * (size_t)len + c;
            if (vec_ok && c + 2 <= len) {
                v = *reinterpret_cast<const double2*>(src);
            } else {
                if (c + 0 < len) v.x = src[0];
                if (c + 1 < len) v.y = src[1];
            }
        }
        r[l] = v;
    }
}

template <int L, int LD, int GROUPS = 64>
__device__ __forceinline__ void stage_store_f64(double (*tile)[LD], const double2 (&r)[L]) {
#pragma unroll
    for (int l = 0; l < L; ++l) {
        const int g = threadIdx.x + 256 * l;
        *reinterpret_cast<double2*>(&tile[g / GROUPS][2 * (g % GROUPS)]) = r[l];
    }
}

// NA: 16-centroid row tiles per pass (8: tiles of 128 centroids; 2 or 4 for up to 32 / 64 clusters).
// A stage copies the 16 NA centroid columns in use; with two row tiles it is 16 features instead
// of 8 (see the fp32 kernel).
template <int NA>
__global__ __launch_bounds__(256, 2) void lloyd_gemm_labels_f64_kernel(
    const double* __restrict__ X_t, const double* __restrict__ centroids_t,
    const double* __restrict__ half_norms, uint32_t* __restrict__ labels,
    const kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k, int x_vec, int c_vec) {
    if (status != nullptr && status->state != KMX_RUNNING) return;
    constexpr int GK = NA == 2 ? 2 * GK64 : GK64;  // features per stage
    constexpr int XL = GK / 4;                     // 128-bit loads per thread and stage, samples
    constexpr int CG = 8 * NA;                     // pairs of columns per centroid row
    constexpr int CL = GK * CG / 256;              // loads per thread and stage, centroids
    constexpr int CLD = 16 * NA + 16;              // row length in doubles: = 16 mod 32, as GLD64
    static_assert(GK * CG % 256 == 0 && CLD % 32 == 16, "whole loads per thread; K rows 32 banks apart");
    __shared__ __align__(16) double xs[2][GK][GLD64];
    __shared__ __align__(16) double cs[2][GK][CLD];
    __shared__ double hn[GT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, j = lane & 15;
    const int n_stages = (d + GK - 1) / GK;
    const int64_t n_tiles = (n + GT - 1) / GT;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * GT;
        double best[2] = {-kmx_inf<double>(), -kmx_inf<double>()};
        int bidx[2] = {0, 0};
        for (int c0 = 0; c0 < k; c0 += 16 * NA) {
            __syncthreads();
            if (threadIdx.x < GT)
                hn[threadIdx.x] = c0 + (int)threadIdx.x < k ? -half_norms[c0 + threadIdx.x] : -kmx_inf<double>();
            double2 rx[XL], rc[CL];
            stage_load_f64<XL>(rx, X_t, n, i0, d, 0, x_vec != 0);
            stage_load_f64<CL, CG>(rc, centroids_t, k, c0, d, 0, c_vec != 0);
            stage_store_f64<XL, GLD64>(xs[0], rx);
            stage_store_f64<CL, CLD, CG>(cs[0], rc);
            __syncthreads();

            // accumulator r of lane (g, j), row tile a, column tile b: centroid 16 a + g + 4 r of
            // sample 32 wave + 16 b + j
            v4d acc[NA][2];
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const double v = hn[16 * a + g + 4 * r];
                    acc[a][0][r] = v;
                    acc[a][1][r] = v;
                }

            for (int st = 0; st < n_stages; ++st) {
                const int cur = st & 1;
                if (st + 1 < n_stages) {
                    stage_load_f64<XL>(rx, X_t, n, i0, d, (st + 1) * GK, x_vec != 0);
                    stage_load_f64<CL, CG>(rc, centroids_t, k, c0, d, (st + 1) * GK, c_vec != 0);
                }
#pragma unroll
                for (int s = 0; s < GK / 4; ++s) {
                    // lane (g, j) supplies feature 4 s + g of centroid / sample j of the 16
                    double bf[2];
#pragma unroll
                    for (int b = 0; b < 2; ++b) bf[b] = xs[cur][4 * s + g][32 * wave + 16 * b + j];
#pragma unroll
                    for (int a = 0; a < NA; ++a) {
                        const double af = cs[cur][4 * s + g][16 * a + j];
#pragma unroll
                        for (int b = 0; b < 2; ++b)
                            acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(af, bf[b], acc[a][b], 0, 0, 0);
                    }
                }
                if (st + 1 < n_stages) {
                    stage_store_f64<XL, GLD64>(xs[cur ^ 1], rx);
                    stage_store_f64<CL, CLD, CG>(cs[cur ^ 1], rc);
                }
                __syncthreads();
            }

#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int c = c0 + 16 * a + g + 4 * r;
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        const double v = acc[a][b][r];
                        if (v > best[b]) {
                            best[b] = v;
                            bidx[b] = c;
                        }
                    }
                }
        }
        // the four lanes of a sample
#pragma unroll
        for (int b = 0; b < 2; ++b) {
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const double ob = __shfl_xor(best[b], off, 64);
                const int oi = __shfl_xor(bidx[b], off, 64);
                if (ob > best[b] || (ob == best[b] && oi < bidx[b])) {
                    best[b] = ob;
                    bidx[b] = oi;
                }
            }
            const int64_t i = i0 + 32 * wave + 16 * b + j;
            if (g == 0 && i < n) labels[i] = (uint32_t)bidx[b];
        }
    }
}

}  // namespace

// Labels of all samples; `half_norms` = 0.5 ||c||^2 per centroid; a null `status` or one in the
// running state lets the kernel work, any other state makes it a no-op.
int32_t kmx_lloyd_gemm_labels(const void* X_t, const void* centroids_t, const void* half_norms,
                              uint32_t* labels, const kmx_lloyd_status* status, int64_t n, int d, int k,
                              int32_t dtype, hipStream_t stream) {
    const size_t s = kmx_dtype_size(dtype);
    const int per_vec = (int)(16 / s);
    auto vec_ok = [&](const void* p, int64_t len) { return (len % per_vec == 0) && ((((uintptr_t)p) & 15) == 0); };
    const int x_vec = vec_ok(X_t, n), c_vec = vec_ok(centroids_t, k);
    int64_t grid = kmx_cdiv(n, GT);
    // workgroups per compute unit: what registers and LDS allow (one workgroup per tile instead
    // measured 4 % slower)
    // (one more with the narrow centroid tiles, whose stages leave the LDS for it)
    const int64_t cap = (int64_t)(dtype == KMX_F32 ? (k > 32 && k <= 64 ? 4 : 3) : (k <= 64 ? 3 : 2)) * kmx_num_cus();
    if (grid > cap) grid = cap;
#define KMX_GEMM_LAUNCH(KERNEL, T)                                                                    \
    hipLaunchKernelGGL(KERNEL, dim3((unsigned)grid), dim3(256), 0, stream, (const T*)X_t,             \
                       (const T*)centroids_t, (const T*)half_norms, labels, status, n, d, k, x_vec, c_vec)
    // centroid tile: 32 / 64 for that few clusters, else 128
    if (dtype == KMX_F32) {
        if (k <= 32) KMX_GEMM_LAUNCH(lloyd_gemm_labels_f32_kernel<1>, float);
        else if (k <= 64) KMX_GEMM_LAUNCH(lloyd_gemm_labels_f32_kernel<2>, float);
        else KMX_GEMM_LAUNCH(lloyd_gemm_labels_f32_kernel<4>, float);
    } else {
        if (k <= 32) KMX_GEMM_LAUNCH(lloyd_gemm_labels_f64_kernel<2>, double);
        else if (k <= 64) KMX_GEMM_LAUNCH(lloyd_gemm_labels_f64_kernel<4>, double);
        else KMX_GEMM_LAUNCH(lloyd_gemm_labels_f64_kernel<8>, double);
    }
#undef KMX_GEMM_LAUNCH
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// The fp32 kernel on the samples list[0 .. *list_count) (both on the device): what a screened
// label kernel could not certify.  The grid covers the worst case; workgroups without a tile
// of the list leave at once.
int32_t kmx_lloyd_gemm_labels_listed(const void* X_t, const void* centroids_t, const void* half_norms,
                                     uint32_t* labels, const kmx_lloyd_status* status, const int* list,
                                     const unsigned int* list_count, int64_t n, int d, int k,
                                     hipStream_t stream) {
    const int c_vec = (k % 4 == 0) && ((((uintptr_t)centroids_t) & 15) == 0);
    int64_t grid = kmx_cdiv(n, GT);
    const int64_t cap = (int64_t)3 * kmx_num_cus();
    if (grid > cap) grid = cap;
#define KMX_GEMM_LISTED(NA_)                                                                                   \
    hipLaunchKernelGGL((lloyd_gemm_labels_f32_kernel<NA_, true>), dim3((unsigned)grid), dim3(256), 0, stream,   \
                       (const float*)X_t, (const float*)centroids_t, (const float*)half_norms, labels, status, \
                       n, d, k, 0, c_vec, list, list_count)
    if (k <= 32) KMX_GEMM_LISTED(1);
    else if (k <= 64) KMX_GEMM_LISTED(2);
    else KMX_GEMM_LISTED(4);
#undef KMX_GEMM_LISTED
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
