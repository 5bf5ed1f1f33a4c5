// fp32 fused Lloyd step on the matrix cores for wide samples / many clusters (e.g.
// n = 1e6, d = 256, k = 1024), where neither the centroids nor (d + 1) * k accumulators fit
// in LDS.
//
//   * A wave owns 32 consecutive samples and keeps ALL their features in registers as the B
//     operands of v_mfma_f32_32x32x2_f32: lane (j, h) holds feature 2s + h of sample j for
//     every K step s (up to 128 VGPRs for d = 256).  X is read from HBM exactly once.
//   * Centroids are the A operand.  The workgroup (4 waves = 128 samples) streams them from
//     L2 in chunks of 128 centroids x 32 features through a double-buffered LDS tile that is a
//     plain row-major copy of the centroids_t sub-block: lane (i, h) reads
//     tile[2s + h][32 b + i], consecutive lanes consecutive addresses.  The next chunk's global
//     loads are in flight while the current chunk is multiplied.
//   * Four centroid blocks (128 centroids) are accumulated at once: four independent MFMA
//     chains, 64 accumulator registers starting at -0.5||c||^2.  After the K loop the arg-max
//     over those 128 centroids costs 192 vector-ALU instructions per 512 MFMAs.
//   * Partial sums.  One global atomic per (sample, feature) would be 2.6e8 atomics per
//     iteration at config 3 (measured: +6 ms on a 4.5 ms kernel).  Instead, when the caller
//     also provides a ROW-MAJOR copy of X, the step only counts samples per cluster; the
//     samples are then bucketed by label (scan + scatter) and one workgroup per bucket chunk
//     sums the bucket's rows - contiguous 4 d-byte reads - in 64-bit fixed point in registers,
//     adding one total per (cluster chunk, feature) to the global sums.  Integer sums do not
//     depend on order, so the result is reproducible.  Without the row-major copy the
//     per-sample atomics are used.  The reduction/finalisation kernels of lloyd.hip follow.
#include "lloyd_layout.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int KC = 32;    // features per LDS chunk (16 K steps)
constexpr int CG = 128;   // centroids per LDS chunk (4 MFMA blocks)

constexpr double FIX_MAGIC = 6755399441055744.0;  // 1.5 * 2^52
constexpr long long FIX_MAGIC_BITS = 0x4338000000000000ll;

__device__ __forceinline__ unsigned long long to_fixed(double scaled_plus_magic) {
    return (unsigned long long)(__double_as_longlong(scaled_plus_magic) - FIX_MAGIC_BITS);
}

// Global loads of one chunk: thread t covers rows t / 32 + 8 q (q = 0..3), columns 4 (t % 32) .. + 3.
// The chunk origin is wave-uniform (scalar base), the thread part a 32-bit offset, so no
// per-chunk 64-bit addresses stay alive across the K loop.
__device__ __forceinline__ void chunk_prefetch(float4 (&regs)[4], const float* __restrict__ centroids_t,
                                               int f0, int c0, int d, int k, bool vec_ok) {
    const int col = (threadIdx.x & 31) * 4;
    const int row0 = threadIdx.x >> 5;
    const float* __restrict__ base = centroids_t + (size_t)f0 * k + c0;  // uniform
    const int c = c0 + col;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = row0 + 8 * q;
        const int off = row * k + col;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (f0 + row < d) {
            if (vec_ok && c + 4 <= k) {
                v = *reinterpret_cast<const float4*>(base + off);
            } else {
                if (c + 0 < k) v.x = base[off + 0];
                if (c + 1 < k) v.y = base[off + 1];
                if (c + 2 < k) v.z = base[off + 2];
                if (c + 3 < k) v.w = base[off + 3];
            }
        }
        regs[q] = v;
    }
}

__device__ __forceinline__ void chunk_store(float (*tile)[CG], const float4 (&regs)[4]) {
    const int col = (threadIdx.x & 31) * 4;
    const int row0 = threadIdx.x >> 5;
#pragma unroll
    for (int q = 0; q < 4; ++q)
        *reinterpret_cast<float4*>(&tile[row0 + 8 * q][col]) = regs[q];
}

constexpr int MODE_LABELS = 0;   // labels only (predict)
constexpr int MODE_ATOMICS = 1;  // labels + one global fixed-point atomic per (sample, feature)
constexpr int MODE_COUNT = 2;    // labels + changed count + per-cluster sample counts; the sums
                                 // are taken afterwards by the bucketed accumulation below

// LISTED: the kernel works on the samples list[0 .. *list_count) instead of 0 .. n - 1 (the
// samples the fp16 screen of lloyd_mfma_wide_screen.hip could not certify) and reads their
// features from the row-major copy X_rm, or gathers them from X_t where there is none.
template <int NKC, int MODE, bool LISTED = false>
__global__ __launch_bounds__(256, 2) void lloyd_mfma_wide_kernel(
    const float* __restrict__ X_t, const float* __restrict__ sample_weight,
    const float* __restrict__ centroids_t, const float* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    kmx_lloyd_status* __restrict__ status, const int* __restrict__ q_exp,
    unsigned long long* __restrict__ gsum, int* __restrict__ counts, int* __restrict__ ranks,
    int64_t n, int d, int k, int vec_ok, const float* __restrict__ X_rm = nullptr,
    const int* __restrict__ list = nullptr, const unsigned int* __restrict__ list_count = nullptr) {
    constexpr bool UPDATE = MODE != MODE_LABELS;
    if (UPDATE && status->state != KMX_RUNNING) return;
    const int64_t n_work = LISTED ? (int64_t)*list_count : n;
    if (LISTED && (int64_t)blockIdx.x * 128 >= n_work) return;

    __shared__ __align__(16) float ctile[2][KC][CG];
    extern __shared__ __align__(16) float hneg_s[];  // [n_cg * CG]: -0.5||c||^2, -inf past k
    __shared__ float scale_s[NKC * KC + 1];          // 2^q per feature, [d] -> weights
    __shared__ unsigned int changed_block;

    const int n_cg = (k + CG - 1) / CG;
    for (int c = threadIdx.x; c < n_cg * CG; c += 256) hneg_s[c] = c < k ? -half_norms[c] : -kmx_inf<float>();
    if (MODE == MODE_ATOMICS) {
        for (int f = threadIdx.x; f <= d; f += 256) scale_s[f] = ldexpf(1.0f, q_exp[f]);
    }
    if (UPDATE && threadIdx.x == 0) changed_block = 0;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int64_t n_tiles = (n_work + 127) >> 7;
    unsigned int changed = 0;
    constexpr int NKS = NKC * 16;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t slot = tile * 128 + wave * 32 + j;
        const bool valid = slot < n_work;
        const int64_t i = LISTED ? (int64_t)list[valid ? slot : 0] : slot;

        // row 2s + h of X_t, advanced by two rows per K step (no per-row offsets kept alive)
        float x[NKS];
        if (LISTED && X_rm != nullptr) {
            const float* __restrict__ xp = X_rm + (size_t)i * d + h;
#pragma unroll
            for (int s = 0; s < NKS; ++s) x[s] = (valid && 2 * s + h < d) ? xp[2 * s] : 0.0f;
        } else {
            // branch-free: out-of-range rows/samples read element 0 of X_t and are zeroed
            const float* __restrict__ xp = X_t + (size_t)h * n + (valid ? i : 0);
            const size_t two_rows = 2 * (size_t)n;
#pragma unroll
            for (int s = 0; s < NKS; ++s) {
                const bool ok = valid && (2 * s + h < d);
                const float v = *(ok ? xp : X_t);
                x[s] = ok ? v : 0.0f;
                xp += two_rows;
            }
        }

        float best = -kmx_inf<float>();
        int code = 0;

        float4 regs[4];
        __syncthreads();  // every wave is done with both LDS buffers (previous tile) and hneg_s is set
        chunk_prefetch(regs, centroids_t, 0, 0, d, k, vec_ok != 0);
        chunk_store(ctile[0], regs);
        __syncthreads();

        for (int cg = 0; cg < n_cg; ++cg) {
            v16f acc[4];
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[b][r] = hneg_s[cg * CG + 32 * b + 8 * (r >> 2) + 4 * h + (r & 3)];

#pragma unroll
            for (int kc = 0; kc < NKC; ++kc) {
                // chunk index within the tile's sequence: cg * NKC + kc; buffer = its parity
                const int step = cg * NKC + kc;
                const bool has_next = (kc + 1 < NKC) || (cg + 1 < n_cg);
                const int next_f0 = (kc + 1 < NKC) ? (kc + 1) * KC : 0;
                const int next_c0 = (kc + 1 < NKC) ? cg * CG : (cg + 1) * CG;
                if (has_next) chunk_prefetch(regs, centroids_t, next_f0, next_c0, d, k, vec_ok != 0);

                // A fragments of K step s + 1 are read from LDS while the MFMAs of step s run;
                // the scheduling barriers keep the compiler from hoisting all 64 reads of the
                // chunk to its top (which costs 64 live registers)
                const float* abase = &ctile[step & 1][h][j];
                float a_cur[4], a_nxt[4];
#pragma unroll
                for (int b = 0; b < 4; ++b) a_cur[b] = abase[32 * b];
#pragma unroll
                for (int s = 0; s < 16; ++s) {
                    if (s + 1 < 16) {
#pragma unroll
                        for (int b = 0; b < 4; ++b) a_nxt[b] = abase[(2 * (s + 1)) * CG + 32 * b];
                    }
                    const float xv = x[kc * 16 + s];
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[b], xv, acc[b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int b = 0; b < 4; ++b) a_cur[b] = a_nxt[b];
                }
                if (has_next) chunk_store(ctile[(step + 1) & 1], regs);
                __syncthreads();
            }

#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int cd = cg * 64 + b * 16 + r;  // wave-uniform
                    if (acc[b][r] > best) {
                        best = acc[b][r];
                        code = cd;
                    }
                }
        }

        // code -> centroid: group (code / 64), block ((code / 16) % 4), register (code % 16)
        int c = CG * (code >> 6) + 32 * ((code >> 4) & 3) + 8 * ((code & 15) >> 2) + 4 * h + (code & 3);
        {
            const float ov = __shfl_xor(best, 32, 64);
            const int oc = __shfl_xor(c, 32, 64);
            if (ov > best || (ov == best && oc < c)) c = oc;
        }
        const uint32_t lab = (uint32_t)c;

        if (valid && h == 0) {
            labels[i] = lab;
            if (UPDATE) changed += (labels_prev[i] != lab) ? 1u : 0u;
            // the returned count is the sample's rank inside its cluster: the scatter that
            // follows needs no atomics of its own
            if (MODE == MODE_COUNT) ranks[i] = atomicAdd(counts + lab, 1);
        }
        if (MODE == MODE_ATOMICS && valid) {
            const double wd = (double)sample_weight[i];
            unsigned long long* dst = gsum + (size_t)h * k + lab;  // row 2s + h, advanced by 2 rows per step
            const float* scp = scale_s + h;
#pragma unroll
            for (int s = 0; s < NKS; ++s) {
                if (2 * s + h < d) {
                    const double sc = (double)scp[2 * s];
                    atomicAdd(dst, to_fixed(fma((double)x[s], wd * sc, FIX_MAGIC)));
                }
                dst += 2 * (size_t)k;
            }
            if (h == 0)
                atomicAdd(gsum + (size_t)d * k + lab, to_fixed(fma(wd, (double)scale_s[d], FIX_MAGIC)));
        }
    }

    if (UPDATE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
    }
}

// ---- bucketed accumulation ---------------------------------------------------------------
// counts[c] samples carry label c and ranks[i] is the position of sample i among them (the
// value its counting atomic returned).  offsets = exclusive scan of counts and
// order[offsets[c] + rank] = the samples of cluster c come from kmx_bucket_order
// (lloyd_bucket.hip); any order will do: the sums below are integers.

// One workgroup per ACC_CHUNK consecutive positions of `order` (samples sorted by cluster),
// whatever the cluster sizes: a workgroup walks the cluster segments inside its range and
// adds one set of totals per segment.  Rows of the ROW-MAJOR copy of X are contiguous: a wave
// reads one whole row per load instruction (lane l takes features 4l .. 4l + 3 as one 128-bit
// load, d <= 256), the four waves of the workgroup take different samples, and every lane
// keeps U loads in flight.  Sums are 64-bit fixed point in registers; the waves' totals are
// combined in LDS and added to the global sums once per segment.  Clears counts for the next
// iteration.
constexpr int ACC_CHUNK = 1024;
constexpr int WIDE_D_MAX = 256;

template <bool VEC>
__global__ __launch_bounds__(256) void bucket_accumulate_kernel(
    const float* __restrict__ X_rm, const float* __restrict__ sample_weight,
    const int* __restrict__ order, const int* __restrict__ offsets, int* __restrict__ counts,
    const int* __restrict__ q_exp, unsigned long long* __restrict__ gsum, int n, int d, int k) {
    __shared__ long long red[4][WIDE_D_MAX + 1];
    __shared__ int c_first;
    const int P0 = blockIdx.x * ACC_CHUNK;
    const int P1 = P0 + ACC_CHUNK < n ? P0 + ACC_CHUNK : n;
    for (int c = blockIdx.x * 256 + threadIdx.x; c < k; c += gridDim.x * 256) counts[c] = 0;
    if (threadIdx.x == 0) c_first = k;
    __syncthreads();
    // the (non-empty) cluster that holds position P0
    for (int c = threadIdx.x; c < k; c += 256)
        if (offsets[c] <= P0 && P0 < offsets[c + 1]) c_first = c;
    __syncthreads();

    constexpr int U = 8;  // rows in flight per lane
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int f4 = lane * 4;
    double sc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sc[j] = f4 + j < d ? (double)ldexpf(1.0f, q_exp[f4 + j]) : 0.0;
    const double sc_w = (double)ldexpf(1.0f, q_exp[d]);
    const float* __restrict__ col = X_rm + (f4 < d ? f4 : 0);

    int c = c_first;
    int pos = P0;
    while (pos < P1 && c < k) {
        const int c_end = offsets[c + 1];  // wave-uniform
        const int p0 = pos, p1 = c_end < P1 ? c_end : P1;
        if (p1 > p0) {
            long long acc[4] = {0, 0, 0, 0};
            long long wsum = 0;
            // each lane fetches one sample index and its weight (one coalesced load + one
            // gather per 64 samples), one group ahead of the rows; lanes past the end hold the
            // last valid sample with weight 0
            auto fetch = [&](int base, int& idx_out, float& w_out) {
                const int pl = base + lane;
                idx_out = order[pl < p1 ? pl : p1 - 1];
                w_out = pl < p1 ? sample_weight[idx_out] : 0.0f;
            };
            int my_idx, next_idx = 0;
            float my_w, next_w = 0.0f;
            fetch(p0, my_idx, my_w);
            for (int base = p0; base < p1; base += 64) {
                if (base + 64 < p1) fetch(base + 64, next_idx, next_w);
                const int n_here = p1 - base < 64 ? p1 - base : 64;
                for (int u0 = wave; u0 < n_here; u0 += 4 * U) {
                    int idx[U];
                    float wv[U];
                    float xv[U][4];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int src = u0 + 4 * u;  // wave-uniform
                        idx[u] = __builtin_amdgcn_readlane(my_idx, src & 63);
                        wv[u] = src < 64 ? __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_w), src & 63)) : 0.0f;
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const float* __restrict__ row = col + (size_t)idx[u] * d;
                        if (VEC) {
                            const float4 v = *reinterpret_cast<const float4*>(row);
                            xv[u][0] = v.x; xv[u][1] = v.y; xv[u][2] = v.z; xv[u][3] = v.w;
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; ++j) xv[u][j] = f4 + j < d ? row[j] : 0.0f;
                        }
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const double wd = (double)wv[u];
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            acc[j] += (long long)to_fixed(fma((double)xv[u][j], wd * sc[j], FIX_MAGIC));
                        wsum += (long long)to_fixed(fma(wd, sc_w, FIX_MAGIC));
                    }
                }
                my_idx = next_idx;
                my_w = next_w;
            }
            // the four waves' totals meet in LDS; one global atomic per feature and segment
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (f4 + j < WIDE_D_MAX) red[wave][f4 + j] = acc[j];
            if (lane == 0) red[wave][WIDE_D_MAX] = wsum;
            __syncthreads();
            for (int f = threadIdx.x; f <= d; f += 256) {
                const int slot = f < d ? f : WIDE_D_MAX;
                const long long tot = (red[0][slot] + red[1][slot]) + (red[2][slot] + red[3][slot]);
                if (tot != 0) atomicAdd(gsum + (size_t)f * k + c, (unsigned long long)tot);
            }
            __syncthreads();
            pos = p1;
        }
        ++c;
    }
}

template <int MODE>
int32_t launch_wide(const LloydLayout& L, const void* X_t, const void* w, const void* centroids_t,
                    const float* half_norms, const uint32_t* labels_prev, uint32_t* labels,
                    kmx_lloyd_status* status, const int* q_exp, unsigned long long* gsum,
                    int* counts, int* ranks, int64_t n, int d, int k, hipStream_t stream) {
    if (!kmx_mfma_wide_supported(d, k)) return KMX_ERR_UNSUPPORTED;
    const int n_cg = (k + CG - 1) / CG;
    const size_t lds = (size_t)n_cg * CG * sizeof(float);
    int64_t grid = kmx_cdiv(n, 128);
    const int64_t cap = 2 * (int64_t)kmx_num_cus();  // register budget allows 2 workgroups per CU
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
    (void)L;
    const int vec_ok = (k % 4 == 0) && ((((uintptr_t)centroids_t) & 15) == 0);
#define KMX_WIDE_CASE(NKC)                                                                      \
    hipLaunchKernelGGL((lloyd_mfma_wide_kernel<NKC, MODE>), dim3((unsigned)grid), dim3(256), lds, \
                       stream, (const float*)X_t, (const float*)w, (const float*)centroids_t,     \
                       half_norms, labels_prev, labels, status, q_exp, gsum, counts, ranks, n, d, k, vec_ok)
    switch ((d + KC - 1) / KC) {
        case 1: KMX_WIDE_CASE(1); break;
        case 2: KMX_WIDE_CASE(2); break;
        case 3: KMX_WIDE_CASE(3); break;
        case 4: KMX_WIDE_CASE(4); break;
        case 5: KMX_WIDE_CASE(5); break;
        case 6: KMX_WIDE_CASE(6); break;
        case 7: KMX_WIDE_CASE(7); break;
        case 8: KMX_WIDE_CASE(8); break;
        default: return KMX_ERR_UNSUPPORTED;
    }
#undef KMX_WIDE_CASE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// One mode on the listed samples only; the grid is fixed because the length of the list is only
// known on the device (blocks without a tile leave at once).
template <int MODE>
int32_t launch_wide_listed(const void* X_t, const void* X_rm, const void* w, const void* centroids_t,
                           const float* half_norms, const uint32_t* labels_prev, uint32_t* labels,
                           kmx_lloyd_status* status, const int* q_exp, unsigned long long* gsum,
                           int* counts, int* ranks, const int* list, const unsigned int* list_count,
                           int64_t n, int d, int k, hipStream_t stream) {
    if (!kmx_mfma_wide_supported(d, k)) return KMX_ERR_UNSUPPORTED;
    const int n_cg = (k + CG - 1) / CG;
    const size_t lds = (size_t)n_cg * CG * sizeof(float);
    int64_t grid = kmx_cdiv(n, 128);
    const int64_t cap = 2 * (int64_t)kmx_num_cus();
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
    const int vec_ok = (k % 4 == 0) && ((((uintptr_t)centroids_t) & 15) == 0);
#define KMX_WIDE_CASE(NKC)                                                                             \
    hipLaunchKernelGGL((lloyd_mfma_wide_kernel<NKC, MODE, true>), dim3((unsigned)grid), dim3(256),       \
                       lds, stream, (const float*)X_t, (const float*)w, (const float*)centroids_t,       \
                       half_norms, labels_prev, labels, status, q_exp, gsum, counts, ranks, n, d, k,     \
                       vec_ok, (const float*)X_rm, list, list_count)
    switch ((d + KC - 1) / KC) {
        case 1: KMX_WIDE_CASE(1); break;
        case 2: KMX_WIDE_CASE(2); break;
        case 3: KMX_WIDE_CASE(3); break;
        case 4: KMX_WIDE_CASE(4); break;
        case 5: KMX_WIDE_CASE(5); break;
        case 6: KMX_WIDE_CASE(6); break;
        case 7: KMX_WIDE_CASE(7); break;
        case 8: KMX_WIDE_CASE(8); break;
        default: return KMX_ERR_UNSUPPORTED;
    }
#undef KMX_WIDE_CASE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

}  // namespace

bool kmx_mfma_wide_supported(int d, int k) {
    // samples live in registers (d <= 256); -0.5||c||^2 of every centroid lives in LDS
    return d <= 256 && k >= 64 && (size_t)((k + CG - 1) / CG) * CG * sizeof(float) <= 28 * 1024;
}

int32_t kmx_lloyd_step_mfma_wide_f32(const LloydLayout& L, const void* X_t, const void* X_rowmajor,
                                     const void* w, const void* centroids_t,
                                     const uint32_t* labels_prev, uint32_t* labels, char* ws,
                                     int64_t n, int d, int k, hipStream_t stream) {
    const int* q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
    auto* status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    auto* gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
    const float* half_norms = reinterpret_cast<const float*>(ws + L.off_half);
    if (X_rowmajor == nullptr || n > INT32_MAX)
        return launch_wide<MODE_ATOMICS>(L, X_t, w, centroids_t, half_norms, labels_prev, labels,
                                         status, q_exp, gsum, nullptr, nullptr, n, d, k, stream);
    // labels + counts, then bucket the samples by label and sum each bucket's rows
    int* counts = reinterpret_cast<int*>(ws + L.off_bucket);
    int* offsets = counts + k;
    int* order = offsets + (k + 1);
    int* ranks = order + n;
    int32_t rc;
    if (kmx_wide_screen_enabled(n, d, k, L.flags)) {
        // labels screened on the fp16 matrix cores; what the screen cannot certify is listed
        // and goes through the all-fp32 kernel
        char* area = ws + L.off_wscreen;
        rc = kmx_lloyd_wide_screen_count(X_t, centroids_t,
                                         reinterpret_cast<const unsigned int*>(ws + L.off_scales), area,
                                         labels_prev, labels, status, counts, ranks, n, d, k, stream);
        if (rc != KMX_OK) return rc;
        rc = launch_wide_listed<MODE_COUNT>(X_t, X_rowmajor, w, centroids_t, half_norms, labels_prev, labels,
                                            status, q_exp, gsum, counts, ranks, kmx_wide_screen_list(area, d, k),
                                            kmx_wide_screen_counter(area), n, d, k, stream);
    } else
        rc = launch_wide<MODE_COUNT>(L, X_t, w, centroids_t, half_norms, labels_prev, labels, status,
                                     q_exp, gsum, counts, ranks, n, d, k, stream);
    if (rc != KMX_OK) return rc;
    rc = kmx_bucket_order(labels, counts, offsets, ranks, order, n, k, stream);
    if (rc != KMX_OK) return rc;
    const unsigned ag = (unsigned)kmx_cdiv(n, ACC_CHUNK);
    if (d % 4 == 0 && ((((uintptr_t)X_rowmajor) & 15) == 0))
        hipLaunchKernelGGL((bucket_accumulate_kernel<true>), dim3(ag), dim3(256), 0, stream,
                           (const float*)X_rowmajor, (const float*)w, order, offsets, counts, q_exp,
                           gsum, (int)n, d, k);
    else
        hipLaunchKernelGGL((bucket_accumulate_kernel<false>), dim3(ag), dim3(256), 0, stream,
                           (const float*)X_rowmajor, (const float*)w, order, offsets, counts, q_exp,
                           gsum, (int)n, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

size_t kmx_assign_wide_screen_bytes(int64_t n, int d, int k, uint32_t flags) {
    if (!kmx_wide_screen_enabled(n, d, k, flags)) return 0;
    return kmx_align256((size_t)d * sizeof(unsigned int)) + kmx_wide_screen_bytes(n, d, k);
}

// Labels only with the fp16 screen: `extra` holds kmx_assign_wide_screen_bytes.  The scale comes
// from the centroids (any scale is a correct one), the listed samples are gathered from X_t.
int32_t kmx_assign_labels_wide_screen_f32(const LloydLayout& L, const void* X_t, const void* centroids_t,
                                          uint32_t* labels, char* ws, char* extra, int64_t n, int d,
                                          int k, hipStream_t stream) {
    unsigned int* absmax = reinterpret_cast<unsigned int*>(extra);
    char* area = extra + kmx_align256((size_t)d * sizeof(unsigned int));
    int32_t rc = kmx_wide_screen_scale_from_centroids(centroids_t, absmax, d, k, stream);
    if (rc != KMX_OK) return rc;
    rc = kmx_lloyd_wide_screen_count(X_t, centroids_t, absmax, area, nullptr, labels, nullptr, nullptr,
                                     nullptr, n, d, k, stream);
    if (rc != KMX_OK) return rc;
    return launch_wide_listed<MODE_LABELS>(X_t, nullptr, nullptr, centroids_t,
                                           reinterpret_cast<const float*>(ws + L.off_half), nullptr, labels,
                                           nullptr, nullptr, nullptr, nullptr, nullptr,
                                           kmx_wide_screen_list(area, d, k), kmx_wide_screen_counter(area),
                                           n, d, k, stream);
}

int32_t kmx_assign_labels_mfma_wide_f32(const LloydLayout& L, const void* X_t,
                                        const void* centroids_t, uint32_t* labels, char* ws,
                                        int64_t n, int d, int k, hipStream_t stream) {
    return launch_wide<MODE_LABELS>(L, X_t, nullptr, centroids_t,
                                    reinterpret_cast<const float*>(ws + L.off_half), nullptr, labels,
                                    nullptr, nullptr, nullptr, nullptr, nullptr, n, d, k, stream);
}
