// The tiled label product of lloyd_gemm.hip for fp32 with the scores SCREENED on the fp16 matrix
// cores and certified per sample, as in lloyd_mfma_screen.hip and lloyd_mfma_wide_screen.hip:
//
//   * X and the centroids are scaled by the power of two that brings max|x| into [2^14, 2^15)
//     and split into two fp16 parts each; score ~ hi*hi + lo*hi + hi*lo accumulated in fp32 from
//     -0.5||c||^2: 3 v_mfma_f32_32x32x16_f16 (96 cycles) per 32 centroids x 32 samples x 16
//     features instead of 8 v_mfma_f32_32x32x2_f32 (512 cycles).
//   * Error of one score (lloyd_mfma_wide_screen.hip has the derivation): with R = 51 roundings
//     per K step of 16 features,
//       E(x) = (7.2e-7 + R 2^-23) ||x|| C + R 2^-23 H + 6.2e-5 sqrt(d) (||x|| + C),
//     C = max ||c||, H = max 0.5||c||^2 in scaled units.  best - second > 2 E(x) certifies the
//     label; any other sample (also one with a non-finite score) goes on a list, and the all-fp32
//     kernel of lloyd_gemm.hip runs on the listed samples afterwards.
//   * A workgroup of four waves owns 128 samples and walks the centroids in tiles of 128 (32 or
//     64 for that few clusters); a stage is 32 features: thread t loads 16 features of one
//     sample and of one centroid (a wave's loads are 256 contiguous bytes of a feature row),
//     scales, splits and stores them as 128-bit operand fragments, [K step][half][index] so
//     that a wave's fragment reads are contiguous.  The next stage's loads are in flight during
//     the MFMAs.  ||x||^2 of the scaled samples is summed on the way (first centroid tile).
//
// An alternative (on request, see kmx_gemm_screen_enabled) for fp32 shapes beyond the other
// screened kernels (more than 64 features with up to 256 clusters, more than 256 features) to
// the label half of fused_lloyd_single_step
// (sklearn_numba_dpex/kmeans/kernels/lloyd_single_step.py:35-424) and assignment
// (kmeans/kernels/compute_labels.py:29-288).
#include "lloyd_layout.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int ST = 128;  // samples per workgroup, centroids per full tile
constexpr int SK = 32;   // features per stage: two K steps of 16

constexpr float GS_ERR_SPLIT = 7.2e-7f;  // 3.01 * 2^-22, rounded up
constexpr float GS_ERR_ROUND = 1.2e-7f;  // 2^-23, rounded up
constexpr float GS_ERR_ABS = 6.2e-5f;    // 2^-14, rounded up

// header words of the screen's area in the workspace
constexpr int GS_HMAX = 0;       // bits of max 0.5||c * scale||^2
constexpr int GS_SCALE = 1;      // bits of the scale
constexpr int GS_UNCERTAIN = 2;  // samples listed by the last label step

// Scale from max|x| per feature (absmax: bits of non-negative floats), max 0.5||c||^2 in scaled
// units, and the list counter cleared.  One workgroup.
__global__ __launch_bounds__(256) void gemm_screen_prep_kernel(const unsigned int* __restrict__ absmax,
                                                               const float* __restrict__ half_norms,
                                                               unsigned int* __restrict__ header, int d, int k) {
    __shared__ float red[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float m = 0.0f;
    for (int f = threadIdx.x; f < d; f += 256) m = fmaxf(m, __uint_as_float(absmax[f]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float xs = (m > 0.0f && m < kmx_inf<float>()) ? ldexpf(1.0f, 14 - ilogbf(m)) : 1.0f;
    __syncthreads();
    float hm = 0.0f;
    for (int c = threadIdx.x; c < k; c += 256) hm = fmaxf(hm, half_norms[c] * xs * xs);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) hm = fmaxf(hm, __shfl_xor(hm, off, 64));
    if (lane == 0) red[wave] = hm;
    __syncthreads();
    if (threadIdx.x == 0) {
        header[GS_HMAX] = __float_as_uint(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
        header[GS_SCALE] = __float_as_uint(xs);
        header[GS_UNCERTAIN] = 0u;
    }
}

// Sixteen features f0 .. f0 + 15 of column `col` of a feature-major array with `len` columns,
// zero outside the array.  One running pointer (a row past the end re-reads the last valid
// address, its value is dropped), so that the sixteen addresses cost no registers.
__device__ __forceinline__ void load16(float (&raw)[16], const float* __restrict__ base, int64_t len,
                                       int64_t col, int d, int f0) {
    const bool col_ok = col < len;
    const int f_first = f0 < d ? f0 : d - 1;
    const float* __restrict__ p = base + (size_t)f_first * (size_t)len + (size_t)(col_ok ? col : 0);
    // all sixteen loads first, the selects afterwards: a select right behind its load makes the
    // compiler wait for every load before it issues the next
    float tmp[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        tmp[e] = *p;
        p += (f0 + e + 1 < d) ? len : 0;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) raw[e] = (col_ok && f0 + e < d) ? tmp[e] : 0.0f;
}

// Scaled values -> fp16 parts, hi = fp16(p), lo = fp16(p - hi) (the subtraction is exact), as
// two 128-bit fragments of eight features each.
template <bool SQ>
__device__ __forceinline__ void split_store(const float (&raw)[16], const float xs, uint4* __restrict__ hi_dst,
                                            uint4* __restrict__ lo_dst, float& sum_sq) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        v8h hi, lo;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = raw[8 * q + e] * xs;
            const _Float16 hb = (_Float16)p;
            hi[e] = hb;
            lo[e] = (_Float16)(p - (float)hb);
            if (SQ) sum_sq = fmaf(p, p, sum_sq);
        }
        hi_dst[q * ST] = __builtin_bit_cast(uint4, hi);
        lo_dst[q * ST] = __builtin_bit_cast(uint4, lo);
    }
}

// NA: 32-centroid row tiles per pass over the features (4: tiles of 128 centroids).
template <int NA>
__global__ __launch_bounds__(256, 2) void lloyd_gemm_screen_f32_kernel(
    const float* __restrict__ X_t, const float* __restrict__ centroids_t,
    const float* __restrict__ half_norms, unsigned int* __restrict__ header, int* __restrict__ list,
    uint32_t* __restrict__ labels, const kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k) {
    if (status != nullptr && status->state != KMX_RUNNING) return;
    // operand fragments: [K step of the stage][half of the K step][sample or centroid]
    __shared__ __align__(16) uint4 xh_s[2][2][ST], xl_s[2][2][ST], ch_s[2][2][ST], cl_s[2][2][ST];
    __shared__ float hn[ST];
    __shared__ float norm_s[ST];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int idx = threadIdx.x & (ST - 1), fg = threadIdx.x >> 7;  // the thread's column and K step of a stage
    const int n_stages = (d + SK - 1) / SK;
    const int64_t n_tiles = (n + ST - 1) / ST;

    const float xs = __uint_as_float(header[GS_SCALE]);
    const float hmax = __uint_as_float(header[GS_HMAX]);
    const float cmax = sqrtf(2.0f * hmax);
    const float round_term = GS_ERR_ROUND * 51.0f * (float)(2 * n_stages);
    const float abs_term = GS_ERR_ABS * sqrtf((float)d);
    const float thr_x = 2.01f * ((GS_ERR_SPLIT + round_term) * cmax + abs_term);
    const float thr_0 = 2.01f * (round_term * hmax + abs_term * cmax);
    const float neg_inf = -kmx_inf<float>();

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * ST;
        float best = neg_inf, second = neg_inf;
        int bidx = 0;
        float sum_sq = 0.0f;
        __syncthreads();  // the previous tile is done with norm_s
        if (threadIdx.x < ST) norm_s[threadIdx.x] = 0.0f;

        for (int c0 = 0; c0 < k; c0 += 32 * NA) {
            const bool first = c0 == 0;
            __syncthreads();  // the previous pass is done with hn and the fragments
            if (threadIdx.x < ST)
                hn[threadIdx.x] = c0 + (int)threadIdx.x < k ? -half_norms[c0 + threadIdx.x] * xs * xs : neg_inf;
            float rx[16], rc[16];
            load16(rx, X_t, n, i0 + idx, d, 16 * fg);
            load16(rc, centroids_t, k, c0 + idx, d, 16 * fg);
            split_store<true>(rx, xs, &xh_s[fg][0][idx], &xl_s[fg][0][idx], sum_sq);
            split_store<false>(rc, xs, &ch_s[fg][0][idx], &cl_s[fg][0][idx], sum_sq);
            __syncthreads();

            // accumulator register r of lane (j, h): centroid 32 a + 8 (r / 4) + 4 h + r % 4
            v16f acc[NA];
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[a][r] = hn[32 * a + 8 * (r >> 2) + 4 * h + (r & 3)];

            for (int st = 0; st < n_stages; ++st) {
                if (st + 1 < n_stages) {
                    load16(rx, X_t, n, i0 + idx, d, (st + 1) * SK + 16 * fg);
                    load16(rc, centroids_t, k, c0 + idx, d, (st + 1) * SK + 16 * fg);
                }
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    // lane (j, h) supplies features 8 h .. 8 h + 7 of the K step, for centroid /
                    // sample j of the 32
                    const v8h xh = __builtin_bit_cast(v8h, xh_s[ks][h][32 * wave + j]);
                    const v8h xl = __builtin_bit_cast(v8h, xl_s[ks][h][32 * wave + j]);
#pragma unroll
                    for (int a = 0; a < NA; ++a) {
                        const v8h ch = __builtin_bit_cast(v8h, ch_s[ks][h][32 * a + j]);
                        const v8h cl = __builtin_bit_cast(v8h, cl_s[ks][h][32 * a + j]);
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ch, xh, acc[a], 0, 0, 0);
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cl, xh, acc[a], 0, 0, 0);
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ch, xl, acc[a], 0, 0, 0);
                    }
                }
                __syncthreads();  // every wave has read the stage
                if (st + 1 < n_stages) {
                    split_store<true>(rx, xs, &xh_s[fg][0][idx], &xl_s[fg][0][idx], sum_sq);
                    split_store<false>(rc, xs, &ch_s[fg][0][idx], &cl_s[fg][0][idx], sum_sq);
                    __syncthreads();
                }
            }

            // best and second best, increasing centroid order per lane, strict comparisons
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float v = acc[a][r];
                    const int c = c0 + 32 * a + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (v > best) {
                        second = best;
                        best = v;
                        bidx = c;
                    } else if (v > second) {
                        second = v;
                    }
                }
            // (summed again in every pass over the features; only the first pass counts)
            if (first) atomicAdd(&norm_s[idx], sum_sq);  // two threads per sample, one per K step
        }
        __syncthreads();
        const float nrm = norm_s[32 * wave + j];

        // the two lanes of a sample: best of both (lower centroid on a tie), second = the larger
        // of the two seconds and the smaller of the two bests
        {
            const float ob = __shfl_xor(best, 32, 64);
            const float o2 = __shfl_xor(second, 32, 64);
            const int oi = __shfl_xor(bidx, 32, 64);
            const float lo_best = ob < best ? ob : best;
            float sec = second > o2 ? second : o2;
            sec = lo_best > sec ? lo_best : sec;
            if (ob > best || (ob == best && oi < bidx)) {
                best = ob;
                bidx = oi;
            }
            second = sec;
        }
        const int64_t i = i0 + 32 * wave + j;
        const bool valid = i < n;
        // written so that a NaN anywhere makes the sample uncertain
        const float thr = fmaf(thr_x, sqrtf(nrm), thr_0);
        const bool unsure = !(best - second > thr) && valid;
        const unsigned long long um = __ballot(h == 0 && unsure);
        if (um) {
            unsigned int base = 0;
            if (lane == 0) base = atomicAdd(header + GS_UNCERTAIN, (unsigned int)__popcll(um));
            base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
            if (h == 0 && unsure) list[base + __popcll(um & ((1ull << lane) - 1ull))] = (int)i;
        }
        if (valid && h == 0) labels[i] = (uint32_t)bidx;  // (provisional for a listed sample)
    }
}

}  // namespace

// Bytes of the screen's area: header (256), then one list entry per sample.
size_t kmx_gemm_screen_bytes(int64_t n) { return 256 + (size_t)n * sizeof(int); }

const uint32_t* kmx_gemm_screen_counter(const char* area) {
    return reinterpret_cast<const uint32_t*>(area) + GS_UNCERTAIN;
}

// Only on request (KMX_FLAG_LABELS_SCREEN): measured against the all-fp32 tiled product it is
// level at 128 features (0.34 ms for 10^6 x 128, 100 clusters) and slower at 768 (the bound
// grows with the number of K steps, 17 % of the samples are then listed, and the in-kernel
// conversion keeps the vector ALU busier than the matrix cores).
bool kmx_gemm_screen_enabled(int64_t n, int d, int k, uint32_t flags) {
    (void)d;
    if (n > INT32_MAX || k < 2) return false;
    return (flags & KMX_FLAG_LABELS_MASK) == KMX_FLAG_LABELS_SCREEN;
}

// Labels of all samples of an fp32 array: screened, then the listed samples in fp32.  `absmax`:
// bits of max|x| per feature (any upper estimate gives correct labels; a poor one lists more
// samples); `area`: kmx_gemm_screen_bytes(n).
int32_t kmx_lloyd_gemm_screen_labels(const void* X_t, const void* centroids_t, const void* half_norms,
                                     const unsigned int* absmax, char* area, uint32_t* labels,
                                     const kmx_lloyd_status* status, int64_t n, int d, int k,
                                     hipStream_t stream) {
    if (n > INT32_MAX) return KMX_ERR_UNSUPPORTED;
    unsigned int* header = reinterpret_cast<unsigned int*>(area);
    int* list = reinterpret_cast<int*>(area + 256);
    hipLaunchKernelGGL(gemm_screen_prep_kernel, dim3(1), dim3(256), 0, stream, absmax, (const float*)half_norms,
                       header, d, k);
    int64_t grid = kmx_cdiv(n, ST);
    const int64_t cap = (int64_t)2 * kmx_num_cus();
    if (grid > cap) grid = cap;
#define KMX_GS_LAUNCH(NA_)                                                                                   \
    hipLaunchKernelGGL((lloyd_gemm_screen_f32_kernel<NA_>), dim3((unsigned)grid), dim3(256), 0, stream,        \
                       (const float*)X_t, (const float*)centroids_t, (const float*)half_norms, header, list, \
                       labels, status, n, d, k)
    if (k <= 32) KMX_GS_LAUNCH(1);
    else if (k <= 64) KMX_GS_LAUNCH(2);
    else KMX_GS_LAUNCH(4);
#undef KMX_GS_LAUNCH
    KMX_LAUNCH_CHECK();
    return kmx_lloyd_gemm_labels_listed(X_t, centroids_t, half_norms, labels, status, list,
                                        header + GS_UNCERTAIN, n, d, k, stream);
}
