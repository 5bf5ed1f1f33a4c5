// Weighted sums per cluster through buckets, for shapes whose (d + 1) * k accumulators do not
// fit in LDS and that the wide fp32 matrix-core path does not cover (fp64, d > 256, few
// clusters of very wide samples).
//
// Replaces, for these shapes, the accumulation half of fused_lloyd_single_step
// (sklearn_numba_dpex/kmeans/kernels/lloyd_single_step.py:35-424), which adds every w * x to
// one of a few global copies of the sums with float atomics.  On this hardware n * d such
// atomics on k * d addresses cost tens of milliseconds per million samples; here the labels
// come from a labels-only kernel, the samples are bucketed by label (counting sort) and each
// bucket's rows are summed in registers, so that global memory sees one atomic per feature and
// per 1024 samples.
//
//   bucket_count   counts[c] and ranks[i] (position of sample i among those of its cluster),
//                  the number of changed labels
//   bucket_offsets offsets = exclusive scan of counts (one workgroup)
//   bucket_scatter order[offsets[label] + rank] = i
//   bucket_sum     one workgroup per 1024 consecutive positions of `order`; a wave takes one
//                  sample at a time with its lanes over the features, so a row of the
//                  row-major copy of X is read as whole cache lines; without that copy the
//                  feature-major array is gathered (a sector per value)
#include "lloyd_layout.h"

namespace {

constexpr int BUCKET_CHUNK = 1024;       // positions of `order` per workgroup of bucket_sum (fewer where the
                                         // array is small: see bucket_sum_chunk)
constexpr int BUCKET_COUNT_TILE = 2048;  // samples per workgroup and pass of bucket_count
constexpr int BUCKET_LDS_K = 4096;       // clusters whose counts are gathered in LDS first

__global__ __launch_bounds__(256) void bucket_count_kernel(
    const uint32_t* __restrict__ labels, const uint32_t* __restrict__ labels_prev,
    int* __restrict__ counts, int* __restrict__ ranks, kmx_lloyd_status* __restrict__ status,
    int64_t n, int k) {
    if (status->state != KMX_RUNNING) return;
    __shared__ int cnt[BUCKET_LDS_K];
    __shared__ unsigned int changed_block;
    const bool in_lds = k <= BUCKET_LDS_K;
    if (threadIdx.x == 0) changed_block = 0;
    unsigned int changed = 0;
    const int64_t n_tiles = (n + BUCKET_COUNT_TILE - 1) / BUCKET_COUNT_TILE;
    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * BUCKET_COUNT_TILE + threadIdx.x;
        constexpr int U = BUCKET_COUNT_TILE / 256;
        uint32_t lab[U];
        int local[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t i = i0 + 256 * u;
            lab[u] = i < n ? labels[i] : 0u;
            changed += (i < n && labels_prev[i] != lab[u]) ? 1u : 0u;
        }
        if (in_lds) {
            // counts of the tile in LDS, one global atomic per cluster present in it
            for (int c = threadIdx.x; c < k; c += 256) cnt[c] = 0;
            __syncthreads();
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (i0 + 256 * u < n) local[u] = atomicAdd(&cnt[lab[u]], 1);
            __syncthreads();
            for (int c = threadIdx.x; c < k; c += 256) {
                const int v = cnt[c];
                if (v != 0) cnt[c] = atomicAdd(&counts[c], v);
            }
            __syncthreads();
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (i0 + 256 * u < n) ranks[i0 + 256 * u] = cnt[lab[u]] + local[u];
            __syncthreads();
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (i0 + 256 * u < n) ranks[i0 + 256 * u] = atomicAdd(&counts[lab[u]], 1);
        }
    }
    if (changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
}

__global__ __launch_bounds__(1024) void bucket_offsets_kernel(const int* __restrict__ counts,
                                                             int* __restrict__ offsets, int k) {
    __shared__ int wave_tot[16];
    __shared__ int carry_s;
    if (threadIdx.x == 0) carry_s = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int c0 = 0; c0 < k; c0 += 1024) {
        const int c = c0 + threadIdx.x;
        const int v = c < k ? counts[c] : 0;
        int incl = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int o = __shfl_up(incl, off, 64);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int base = carry_s;
        for (int w2 = 0; w2 < wave; ++w2) base += wave_tot[w2];
        if (c < k) offsets[c] = base + incl - v;
        __syncthreads();
        if (threadIdx.x == 1023) carry_s = base + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) offsets[k] = carry_s;
}

__global__ __launch_bounds__(256) void bucket_scatter_kernel(const uint32_t* __restrict__ labels,
                                                             const int* __restrict__ offsets,
                                                             const int* __restrict__ ranks,
                                                             int* __restrict__ order, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        order[offsets[labels[i]] + ranks[i]] = (int)i;
}

__device__ __forceinline__ double read_lane(double v, int src) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_readlane((int)(b & 0xffffffffLL), src);
    const int hi = __builtin_amdgcn_readlane((int)(b >> 32), src);
    return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}

// ROW_MAJOR: X is the n x d copy (a sample's features are contiguous), else the d x n array.
// Sums are taken in fp64 whatever T is; the workgroup adds one total per feature and per
// cluster segment of its chunk to `sums` ((d + 1) x k, feature-major, the weights last).
// Clears counts for the next iteration.  NJ: features per lane and pass (64 NJ features per
// pass; one for arrays of up to 64 features, which then pay for one load and one product per
// lane and sample and not for four).
template <typename T, bool ROW_MAJOR, int NJ>
__global__ __launch_bounds__(256) void bucket_sum_kernel(
    const T* __restrict__ X, const T* __restrict__ sample_weight, const int* __restrict__ order,
    const int* __restrict__ offsets, int* __restrict__ counts, T* __restrict__ sums,
    const kmx_lloyd_status* __restrict__ status, int n, int d, int k, int chunk) {
    if (status->state != KMX_RUNNING) return;
    constexpr int FB = 64 * NJ;  // features per pass
    __shared__ double red[4][FB + 1];
    __shared__ int c_first;
    // (a chunk of `chunk` positions per workgroup, and the passes over the features dealt out over
    // the second grid dimension)
    const int P0 = blockIdx.x * chunk;
    const int P1 = P0 + chunk < n ? P0 + chunk : n;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < k; c += gridDim.x * 256) counts[c] = 0;
    if (threadIdx.x == 0) c_first = k;
    __syncthreads();
    // the (non-empty) cluster that holds position P0
    for (int c = threadIdx.x; c < k; c += 256)
        if (offsets[c] <= P0 && P0 < offsets[c + 1]) c_first = c;
    __syncthreads();

    constexpr int U = 4;  // samples in flight per wave
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    for (int fb = (int)blockIdx.y * FB; fb < d; fb += (int)gridDim.y * FB) {
        size_t col[NJ];   // the lane's features of this pass (clamped: past d the value is dropped)
        bool live[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int f = fb + lane + 64 * j;
            live[j] = f < d;
            const int fc = live[j] ? f : d - 1;
            col[j] = ROW_MAJOR ? (size_t)fc : (size_t)fc * (size_t)n;
        }
        int c = c_first;
        int pos = P0;
        while (pos < P1 && c < k) {
            const int c_end = offsets[c + 1];  // wave-uniform
            const int p0 = pos, p1 = c_end < P1 ? c_end : P1;
            if (p1 > p0) {
                double acc[NJ];
#pragma unroll
                for (int j = 0; j < NJ; ++j) acc[j] = 0.0;
                double wsum = 0.0;
                // each lane fetches one sample index and its weight (a coalesced load and a
                // gather per 64 samples); lanes past the end hold the last sample, weight 0
                for (int base = p0; base < p1; base += 64) {
                    const int pl = base + lane;
                    const int my_idx = order[pl < p1 ? pl : p1 - 1];
                    const double my_w = pl < p1 ? (double)sample_weight[my_idx] : 0.0;
                    const int n_here = p1 - base < 64 ? p1 - base : 64;
                    for (int u0 = wave; u0 < n_here; u0 += 4 * U) {
                        T xv[U][NJ];
                        double wv[U];
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            const int src = u0 + 4 * u;  // wave-uniform; past the end: weight 0
                            const int idx = __builtin_amdgcn_readlane(my_idx, src & 63);
                            wv[u] = src < n_here ? read_lane(my_w, src & 63) : 0.0;
                            const T* __restrict__ row = ROW_MAJOR ? X + (size_t)idx * (size_t)d : X + idx;
#pragma unroll
                            for (int j = 0; j < NJ; ++j) xv[u][j] = row[col[j]];
                        }
#pragma unroll
                        for (int u = 0; u < U; ++u) {
#pragma unroll
                            for (int j = 0; j < NJ; ++j) acc[j] = fma((double)xv[u][j], wv[u], acc[j]);
                            wsum += wv[u];
                        }
                    }
                }
                // the four waves' totals meet in LDS; one global atomic per feature and segment
#pragma unroll
                for (int j = 0; j < NJ; ++j) red[wave][lane + 64 * j] = live[j] ? acc[j] : 0.0;
                if (lane == 0) red[wave][FB] = wsum;
                __syncthreads();
                {
                    const int f = fb + (int)threadIdx.x;
                    if (f < d) {
                        const double tot = (red[0][threadIdx.x] + red[1][threadIdx.x]) +
                                           (red[2][threadIdx.x] + red[3][threadIdx.x]);
                        if (tot != 0.0) kmx_atomic_add(sums + (size_t)f * k + c, (T)tot);
                    }
                    if (fb == 0 && threadIdx.x == 0) {
                        const double tot = (red[0][FB] + red[1][FB]) + (red[2][FB] + red[3][FB]);
                        if (tot != 0.0) kmx_atomic_add(sums + (size_t)d * k + c, (T)tot);
                    }
                }
                __syncthreads();
                pos = p1;
            }
            ++c;
        }
    }
}


// ---------------------------------------------------------------------------- sums without buckets
// fp32, every cluster's sums within one workgroup's LDS as 64-bit fixed point (the scales are
// those of the fused matrix-core steps: term = round(x * w * 2^q_f), so that the sums do not
// depend on the order of the additions): a thread takes a sample, reads its label, and adds its
// features with LDS atomics; the workgroup then adds its accumulators to the global ones.  One
// pass over X_t in its own order, no sorting of the samples, one launch instead of four.
constexpr int DS_THREADS = 1024;
constexpr int DS_AHEAD = 8;  // features of a sample in flight together

// 1.5 * 2^(52 - q): adding it to |v| < 2^(51 - q) leaves round-to-nearest(v * 2^q) in the low
// mantissa bits (the low word of the constant is zero).
__device__ __forceinline__ double ds_magic(int q) {
    return __hiloint2double((int)(0x43380000u - ((unsigned int)q << 20)), 0);
}
__device__ __forceinline__ unsigned long long ds_fixed(double v_plus_magic, double magic) {
    return (unsigned long long)(__double_as_longlong(v_plus_magic) - __double_as_longlong(magic));
}

__global__ __launch_bounds__(DS_THREADS) void direct_sums_kernel(
    const float* __restrict__ X_t, const float* __restrict__ w, const uint32_t* __restrict__ labels_prev,
    const uint32_t* __restrict__ labels, const int* __restrict__ q_exp,
    unsigned long long* __restrict__ gsum, kmx_lloyd_status* __restrict__ status, int n, int d, int k) {
    if (status->state != KMX_RUNNING) return;
    extern __shared__ unsigned long long ds_acc[];  // (d + 1, k), feature-major like gsum
    __shared__ int q_s[65];
    __shared__ unsigned int changed_block;
    const int items = (d + 1) * k;
    for (int j = threadIdx.x; j < items; j += DS_THREADS) ds_acc[j] = 0ull;
    if (threadIdx.x <= d) q_s[threadIdx.x] = q_exp[threadIdx.x];
    if (threadIdx.x == 0) changed_block = 0u;
    __syncthreads();
    unsigned int changed = 0u;
    for (int64_t base = (int64_t)blockIdx.x * DS_THREADS; base < n; base += (int64_t)gridDim.x * DS_THREADS) {
        const int64_t i = base + threadIdx.x;
        const bool live = i < n;
        const int64_t ic = live ? i : n - 1;
        const uint32_t lab = labels[ic];
        changed += (live && labels_prev[ic] != lab) ? 1u : 0u;
        const double wd = live ? (double)w[ic] : 0.0;
        unsigned long long* mine = ds_acc + lab;
        for (int f0 = 0; f0 < d; f0 += DS_AHEAD) {
            float xv[DS_AHEAD];
#pragma unroll
            for (int u = 0; u < DS_AHEAD; ++u) {
                const int f = f0 + u < d ? f0 + u : d - 1;  // (uniform; the repeats are not added)
                xv[u] = X_t[(size_t)f * n + ic];
            }
#pragma unroll
            for (int u = 0; u < DS_AHEAD; ++u)
                if (f0 + u < d) {
                    const double magic = ds_magic(q_s[f0 + u]);
                    // x * w is exact in fp64; one rounding, to a multiple of 2^-q
                    const unsigned long long term = ds_fixed(fma((double)xv[u], wd, magic), magic);
                    if (live) atomicAdd(mine + (size_t)(f0 + u) * k, term);
                }
        }
        if (live) {
            const double magic_w = ds_magic(q_s[d]);
            atomicAdd(mine + (size_t)d * k, ds_fixed(wd + magic_w, magic_w));
        }
    }
    if (changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
    // every workgroup starts at another word: they finish together and would otherwise queue up
    // on the same addresses
    const int rot = (int)(((int64_t)blockIdx.x * items) / gridDim.x);
    for (int jy = threadIdx.x; jy < items; jy += DS_THREADS) {
        const int jx = jy + rot < items ? jy + rot : jy + rot - items;
        const unsigned long long v = ds_acc[jx];
        if (v) atomicAdd(gsum + jx, v);
    }
}

}  // namespace

size_t kmx_bucket_bytes(int64_t n, int k) { return ((size_t)2 * k + 1 + 2 * (size_t)n) * sizeof(int); }

// offsets and order from counts and ranks (also used by the wide fp32 path)
int32_t kmx_bucket_order(const uint32_t* labels, const int* counts, int* offsets, const int* ranks,
                         int* order, int64_t n, int k, hipStream_t stream) {
    hipLaunchKernelGGL(bucket_offsets_kernel, dim3(1), dim3(1024), 0, stream, counts, offsets, k);
    int64_t sg = kmx_cdiv(n, 256 * 4);
    if (sg > 2048) sg = 2048;
    hipLaunchKernelGGL(bucket_scatter_kernel, dim3((unsigned)sg), dim3(256), 0, stream, labels, offsets, ranks,
                       order, n);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// After a labels-only kernel: sums[(d + 1) * k] += the weighted rows per cluster, and
// status->n_changed.  `bucket` holds kmx_bucket_bytes; its first k words (the counts) are zero on
// entry and on return.
int32_t kmx_lloyd_bucket_sums(const void* X_t, const void* X_rowmajor, const void* w,
                              const uint32_t* labels_prev, const uint32_t* labels, void* sums,
                              kmx_lloyd_status* status, char* bucket, int64_t n, int d, int k,
                              int32_t dtype, hipStream_t stream) {
    if (n > INT32_MAX) return KMX_ERR_UNSUPPORTED;
    int* counts = reinterpret_cast<int*>(bucket);
    int* offsets = counts + k;
    int* order = offsets + (k + 1);
    int* ranks = order + n;
    int64_t cg = kmx_cdiv(n, BUCKET_COUNT_TILE);
    const int64_t cap = (int64_t)8 * kmx_num_cus();
    if (cg > cap) cg = cap;
    hipLaunchKernelGGL(bucket_count_kernel, dim3((unsigned)cg), dim3(256), 0, stream, labels, labels_prev,
                       counts, ranks, status, n, k);
    KMX_LAUNCH_CHECK();
    const int32_t rc = kmx_bucket_order(labels, counts, offsets, ranks, order, n, k, stream);
    if (rc != KMX_OK) return rc;
    // With few samples a chunk of 1024 positions per workgroup leaves most compute units without
    // one (10^5 samples: 98 workgroups): smaller chunks, down to 128 positions, and the passes over
    // the features side by side, until there are about four workgroups per compute unit.
    const int64_t want = (int64_t)4 * kmx_num_cus();
    int chunk = BUCKET_CHUNK;
    while (chunk > 128 && kmx_cdiv(n, chunk) < want) chunk >>= 1;
    const unsigned ag = (unsigned)kmx_cdiv(n, chunk);
    const int fb_features = d <= 64 ? 64 : d <= 128 ? 128 : 256;
    int64_t gy = kmx_cdiv(want, ag);
    if (gy > kmx_cdiv(d, fb_features)) gy = kmx_cdiv(d, fb_features);
    if (gy < 1) gy = 1;
#define KMX_BUCKET_SUM_NJ(T, RM, XP, NJ_)                                                                \
    hipLaunchKernelGGL((bucket_sum_kernel<T, RM, NJ_>), dim3(ag, (unsigned)gy), dim3(256), 0, stream,   \
                       (const T*)(XP), (const T*)w, order, offsets, counts, (T*)sums, status, (int)n, d, k, chunk)
#define KMX_BUCKET_SUM(T, RM, XP)                      \
    do {                                               \
        if (d <= 64) KMX_BUCKET_SUM_NJ(T, RM, XP, 1);  \
        else if (d <= 128) KMX_BUCKET_SUM_NJ(T, RM, XP, 2); \
        else KMX_BUCKET_SUM_NJ(T, RM, XP, 4);          \
    } while (0)
    if (dtype == KMX_F32) {
        if (X_rowmajor != nullptr) KMX_BUCKET_SUM(float, true, X_rowmajor);
        else KMX_BUCKET_SUM(float, false, X_t);
    } else {
        if (X_rowmajor != nullptr) KMX_BUCKET_SUM(double, true, X_rowmajor);
        else KMX_BUCKET_SUM(double, false, X_t);
    }
#undef KMX_BUCKET_SUM
#undef KMX_BUCKET_SUM_NJ
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// The sums of kmx_lloyd_direct_sums fit one workgroup's LDS (160 KB on this hardware, some of it
// left to the kernel's own words).
bool kmx_direct_sums_fits(int d, int k) {
    return d <= 64 && (size_t)(d + 1) * k * sizeof(unsigned long long) <= (size_t)150 * 1024;
}

// Adds sum w x per cluster (and sum w in row d) to the fixed-point sums `gsum` ((d + 1, k), scales
// `q_exp` as prepared for the fused matrix-core steps) and the number of changed labels to the
// status; fp32 only.
int32_t kmx_lloyd_direct_sums(const void* X_t, const void* w, const uint32_t* labels_prev,
                              const uint32_t* labels, const int* q_exp, unsigned long long* gsum,
                              kmx_lloyd_status* status, int64_t n, int d, int k, hipStream_t stream) {
    if (!kmx_direct_sums_fits(d, k) || n > INT32_MAX || n < 1) return KMX_ERR_UNSUPPORTED;
    const size_t lds = (size_t)(d + 1) * k * sizeof(unsigned long long);
    if (lds > 64 * 1024) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&direct_sums_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int32_t)e;
    }
    int64_t grid = kmx_cdiv(n, DS_THREADS);
    const int cus = kmx_num_cus();
    if (grid > cus) grid = cus;
    hipLaunchKernelGGL(direct_sums_kernel, dim3((unsigned)grid), dim3(DS_THREADS), lds, stream,
                       (const float*)X_t, (const float*)w, labels_prev, labels, q_exp, gsum, status, (int)n,
                       d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
