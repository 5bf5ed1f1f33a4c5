// kmeans++ seeding for gfx950, with no host round trip between centres.
//
// State lives in a caller-provided workspace:
//   header      best row of the last step, total potential of that row
//   candidates  2 x 16 int32 (two buffers so that a fused select+sample launch can read the
//               previous candidates while it writes the next ones)
//   potentials  16 doubles (row sums of the last step)
//   block_pot   (n_blocks, 16) doubles: per-workgroup partial row sums; workgroup b owns the
//               samples [b * 1024, (b + 1) * 1024), so these are also the coarse level of the
//               sampler's two-level search
//   cand_rows   (16, d): the feature rows of the current candidates, copied when they are
//               sampled so that the step kernel reads them with wave-uniform (scalar) loads
//   rows        (n_trials, n) in the compute dtype: min(w * ||x - x_cand||^2, closest) for
//               every candidate; `closest` IS the best row, updated in place: a thread reads
//               closest[i] before it writes column i of every row.
//
// Per new centre: [select previous best + sample candidates] then [step].  The sampler is a
// search in the fp64 inclusive scan of `closest`: coarse over the block sums, fine inside one
// block of 1024 samples, so it never re-reads the whole array.
#include "kmx_common.h"

#include <type_traits>

namespace {

constexpr int TN_MAX = 16;      // n_local_trials = 2 + floor(ln k) <= 16 for k < 1.2e6
constexpr int CHUNK = 1024;     // samples per workgroup (256 threads x 4)
constexpr int SPLIT_MIN_D = 64; // from this many features on, few samples are stepped with the
                                // features split over the four waves of a workgroup

struct KppHeader {
    int32_t best_row;
    int32_t pad;
    double total;
};

struct KppLayout {
    size_t off_header, off_cand, off_pot, off_cand_rows, off_block_pot, off_rows, total;
    int64_t n_blocks;
    int chunk;  // samples per block sum: CHUNK, or 64 * split
    int split;  // 0, or the samples per thread (1, 2, 4) of the feature-split step kernel
};

// Samples per thread of the feature-split step kernel, 0 when the shape keeps the plain one.
// With CHUNK samples per workgroup a short, wide array gives the chip a few dozen workgroups
// that each walk every feature; 64 * split samples per workgroup and a quarter of the features
// per wave give it thousands of waves.  The block sums stay at most 1 024, which the selection
// kernel keeps in registers.
int kpp_split(int64_t n, int d, int n_trials, int dtype) {
    if (d < SPLIT_MIN_D) return 0;
    // (the partial distances of a workgroup: 4 waves x trials x samples, at most 32 KB)
    const int most = (dtype == KMX_F32 ? 4 : 2) / (n_trials > 8 ? 2 : 1);
    const int spt = n <= 65536 ? 1 : n <= 131072 ? 2 : n <= 262144 ? 4 : 8;
    return spt <= most ? spt : 0;
}

// The layout, the block sums included, depends on the shape only: calls with either sampler
// may follow one another on one workspace.
KppLayout kpp_layout(int64_t n, int d, int n_trials, int dtype) {
    KppLayout L;
    L.split = kpp_split(n, d, n_trials, dtype);
    L.chunk = L.split ? 64 * L.split : CHUNK;
    L.n_blocks = kmx_cdiv(n, L.chunk);
    L.off_header = 0;
    L.off_cand = 256;
    L.off_pot = 512;
    L.off_cand_rows = 768;  // (TN_MAX, d): the candidates' feature rows, read by the step kernel a batch at a time
    L.off_block_pot = L.off_cand_rows + kmx_align256((size_t)TN_MAX * d * kmx_dtype_size(dtype));
    L.off_rows = L.off_block_pot + kmx_align256((size_t)L.n_blocks * TN_MAX * sizeof(double));
    L.total = L.off_rows + kmx_align256((size_t)n_trials * n * kmx_dtype_size(dtype));
    return L;
}

// acc + diff^2.  FUSED: one rounding (fused multiply-add), the default.  Not FUSED: product and
// sum rounded separately, the two statements of the reference's kernels taken literally
// (kmeans/kernels/kmeans_plusplus.py:44-48, 226-230); the literal sampler's running sum in the
// compute dtype amplifies a last-bit difference in one distance into another candidate, so
// the literal mode has to reproduce the distances bit for bit as well.
template <bool FUSED, typename T>
__device__ __forceinline__ T kpp_sq_acc(T diff, T acc) {
    if constexpr (FUSED) {
        return fma(diff, diff, acc);
    } else {
#pragma clang fp contract(off)
        const T p = diff * diff;
        return acc + p;
    }
}

// Four consecutive values of a row at i0 (one or two 128-bit accesses when `full`), zero past n.
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

// The value lane `src` (a constant) holds, as a wave-uniform scalar.
template <typename T>
__device__ __forceinline__ T kpp_readlane(T v, int src) {
    if constexpr (sizeof(T) == 4) {
        return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
    } else {
        const long long b = __double_as_longlong(v);
        const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)b, src);
        const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(b >> 32), src);
        return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
    }
}

// The candidates' values of one batch of FB features, fetched with the samples' own loads:
// lane l of load q asks for feature f0 + l % FB of trial q * (64 / FB) + l / FB (indices
// clamped to the rows in use), and the feature loop reads each value back from its lane as a
// scalar.  One scalar load per value, each waited for where it is used, took a round trip
// per candidate and feature instead.
template <typename T, int TN, int FB>
struct KppCandBatch {
    static constexpr int TPL = 64 / FB;  // trials per load
    static constexpr int NQ = (TN + TPL - 1) / TPL;
    T v[NQ];
    __device__ __forceinline__ void load(const T* __restrict__ cand_rows, int f0, int d, int n_trials, int lane) {
        const int f = f0 + lane % FB < d ? f0 + lane % FB : d - 1;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int t = q * TPL + lane / FB;
            v[q] = cand_rows[(size_t)(t < n_trials ? t : n_trials - 1) * d + f];
        }
    }
    __device__ __forceinline__ T get(int t, int j) const { return kpp_readlane<T>(v[t / TPL], (t % TPL) * FB + j); }
};

// rows[t, i] = min(w_i * ||x_i - x_cand_t||^2, closest_i) and per-block row sums.
// Candidate rows come from a small (TN, d) buffer, a batch of features at a time spread over
// the lanes and read back as scalars (no LDS, no barriers in the feature loop); every thread
// streams 4 consecutive samples of a batch of features with 128-bit loads.
// INIT: the first distances instead, closest = w * ||x - x_start||^2 into row 0 with its block
// sums, and slot 0 of the outputs: one trial whose candidate is sample `start`, no minimum.
template <typename T, int TN, bool FUSED, bool INIT>
__global__ __launch_bounds__(256) void kpp_step_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight, const T* __restrict__ cand_rows,
    T* __restrict__ rows, double* __restrict__ block_pot, KppHeader* __restrict__ header,
    int64_t n, int d, int k, int n_trials, int vec_ok, int32_t start, T* __restrict__ centers_t,
    int32_t* __restrict__ center_indices) {
    __shared__ double wave_pot[4][TN];
    const int64_t i0 = (int64_t)blockIdx.x * CHUNK + threadIdx.x * 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int best = INIT ? 0 : header->best_row;
    // Whether the 128-bit accesses are legal is decided once per workgroup and known at compile
    // time inside the body: with a test per access every load sat in a branch of its own and
    // was waited for before the next one was issued.
    auto body = [&](auto full_tag) {
    constexpr bool full = decltype(full_tag)::value;

    // weights and the closest distances so far are needed after the feature loop: requested
    // with its last batch
    T w[4], cl[4];

    T acc[TN][4];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[t][r] = T(0);

    // Features in batches of FB rows: 16 loads of 16 bytes per lane in flight at a time in fp32
    // (a wave has 64 KB to stream and only four of them share a SIMD).
    constexpr int FB = sizeof(T) == 4 ? 16 : 8;
    for (int f0 = 0; f0 < d; f0 += FB) {
        T xv[FB][4];
#pragma unroll
        for (int j = 0; j < FB; ++j) {
            const int f = f0 + j < d ? f0 + j : d - 1;  // past the end: a valid row, ignored below
            const T* __restrict__ row = X_t + (size_t)f * n;
            load4<T>(row, i0, n, full, xv[j]);
        }
        KppCandBatch<T, TN, FB> cand;
        if constexpr (INIT) {
            const int f = f0 + lane % FB < d ? f0 + lane % FB : d - 1;
            cand.v[0] = X_t[(size_t)f * n + start];
        } else {
            cand.load(cand_rows, f0, d, n_trials, lane);
        }
        if (f0 + FB >= d) {
            load4<T>(sample_weight, i0, n, full, w);
            if constexpr (!INIT) load4<T>(rows + (size_t)best * n, i0, n, full, cl);
        }
        auto accumulate = [&](auto whole_tag) {
            constexpr bool whole = decltype(whole_tag)::value;  // all FB features exist
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                if (t < n_trials) {
#pragma unroll
                    for (int j = 0; j < FB; ++j) {
                        if (whole || f0 + j < d) {
                            const T cv = cand.get(t, j);
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                const T diff = xv[j][r] - cv;
                                acc[t][r] = kpp_sq_acc<FUSED>(diff, acc[t][r]);
                            }
                        }
                    }
                }
            }
        };
        if (f0 + FB <= d)
            accumulate(std::true_type{});
        else
            accumulate(std::false_type{});
    }

    double pot[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        pot[t] = 0.0;
        if (t < n_trials) {
            T v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                v[r] = acc[t][r] * w[r];
                if constexpr (!INIT) v[r] = fmin(v[r], cl[r]);
                if (i0 + r < n) pot[t] += (double)v[r];
            }
            store4<T>(rows + (size_t)t * n, i0, n, full, v);
        }
    }
    // all row sums of the workgroup with one barrier: waves first, then one thread per trial
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        if (t < n_trials) {
            const double ws = kmx_wave_sum<double>(pot[t]);
            if (lane == 0) wave_pot[wave][t] = ws;
        }
    }
    __syncthreads();
    if (threadIdx.x < n_trials)
        block_pot[(size_t)blockIdx.x * TN_MAX + threadIdx.x] =
            (wave_pot[0][threadIdx.x] + wave_pot[1][threadIdx.x]) +
            (wave_pot[2][threadIdx.x] + wave_pot[3][threadIdx.x]);
    };
    if (vec_ok && (int64_t)(blockIdx.x + 1) * CHUNK <= n)
        body(std::true_type{});
    else
        body(std::false_type{});
    if (INIT && blockIdx.x == 0) {
        for (int f = threadIdx.x; f < d; f += 256) centers_t[(size_t)f * k] = X_t[(size_t)f * n + start];
        if (threadIdx.x == 0) {
            center_indices[0] = start;
            header->best_row = 0;
            header->total = 0.0;
        }
    }
}

// SPT consecutive values of a row at i0: one access of SPT elements when `full`, else element
// by element from indices clamped to the array (the caller ignores what lies past n).
template <typename T, int SPT>
__device__ __forceinline__ void load_spt(const T* __restrict__ row, int64_t i0, int64_t n, bool full, T (&v)[SPT]) {
    if (full) {
        if constexpr (SPT == 1) {
            v[0] = row[i0];
        } else if constexpr (SPT == 2) {
            using V2 = std::conditional_t<sizeof(T) == 4, float2, double2>;
            const V2 q = *reinterpret_cast<const V2*>(row + i0);
            v[0] = q.x; v[1] = q.y;
        } else {
            load4<T>(row, i0, n, true, v);
        }
    } else {
#pragma unroll
        for (int r = 0; r < SPT; ++r) v[r] = row[i0 + r < n ? i0 + r : n - 1];
    }
}

// The step (or, INIT, the first distances to the starting sample) for few samples of many
// features.  A workgroup owns 64 * SPT samples; its four waves take the feature batches in
// turn, every lane streaming SPT consecutive samples, and leave partial squared distances in
// LDS.  After one barrier wave w finishes trials w, w + 4: the four partial sums added in wave
// order, weight, minimum with the closest distance so far, the row store and the block sum.
// The closest distances are read before the barrier: the finishing waves overwrite the row
// they came from.  LITERAL keeps the reference's roundings (features summed in order, product
// and sum rounded separately): every wave walks all the features and the first one's sums are
// used, so that the block sums have one geometry for both samplers.
template <typename T, int TN, int SPT, bool INIT, bool LITERAL>
__global__ __launch_bounds__(256) void kpp_step_split_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight, const T* __restrict__ cand_rows,
    T* __restrict__ rows, double* __restrict__ block_pot, KppHeader* __restrict__ header, int64_t n,
    int d, int k, int n_trials, int vec_ok, int32_t start, T* __restrict__ centers_t,
    int32_t* __restrict__ center_indices) {
    constexpr int S = 64 * SPT;
    __shared__ T part[4][TN][S];
    // the wave index as a scalar: the feature loop's bounds and the candidates' rows are then
    // wave-uniform for the compiler as well (scalar branches, no lane masks per feature)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t base = (int64_t)blockIdx.x * S;
    const int64_t i0 = base + lane * SPT;
    const int best = INIT ? 0 : header->best_row;

    // what the finish needs of samples base + r * 64 + lane, requested ahead of the feature loop
    T w_fin[SPT], cl_fin[SPT];
#pragma unroll
    for (int r = 0; r < SPT; ++r) {
        const int64_t i = base + r * 64 + lane;
        const int64_t ic = i < n ? i : n - 1;
        w_fin[r] = sample_weight[ic];
        cl_fin[r] = INIT ? T(0) : rows[(size_t)best * n + ic];
    }

    auto body = [&](auto full_tag) {
        constexpr bool full = decltype(full_tag)::value;
        T acc[TN][SPT];
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int r = 0; r < SPT; ++r) acc[t][r] = T(0);
        constexpr int FB = sizeof(T) == 4 ? 16 : 8;
        for (int f0 = LITERAL ? 0 : wave * FB; f0 < d; f0 += LITERAL ? FB : 4 * FB) {
            T xv[FB][SPT];
#pragma unroll
            for (int j = 0; j < FB; ++j) {
                const int f = f0 + j < d ? f0 + j : d - 1;  // past the end: a valid row, ignored below
                load_spt<T, SPT>(X_t + (size_t)f * n, i0, n, full, xv[j]);
            }
            // the candidates' rows, or the starting sample's features
            KppCandBatch<T, TN, FB> cand;
            if constexpr (INIT) {
                const int f = f0 + lane % FB < d ? f0 + lane % FB : d - 1;
                cand.v[0] = X_t[(size_t)f * n + start];
            } else {
                cand.load(cand_rows, f0, d, n_trials, lane);
            }
            auto accumulate = [&](auto whole_tag) {
                constexpr bool whole = decltype(whole_tag)::value;  // all FB features exist
#pragma unroll
                for (int t = 0; t < TN; ++t) {
                    if (t < n_trials) {
#pragma unroll
                        for (int j = 0; j < FB; ++j) {
                            if (whole || f0 + j < d) {
                                const T cv = cand.get(t, j);
#pragma unroll
                                for (int r = 0; r < SPT; ++r) {
                                    const T diff = xv[j][r] - cv;
                                    acc[t][r] = kpp_sq_acc<!LITERAL>(diff, acc[t][r]);
                                }
                            }
                        }
                    }
                }
            };
            if (f0 + FB <= d)
                accumulate(std::true_type{});
            else
                accumulate(std::false_type{});
        }
#pragma unroll
        for (int t = 0; t < TN; ++t)
            if (t < n_trials)
#pragma unroll
                for (int r = 0; r < SPT; ++r) part[wave][t][lane * SPT + r] = acc[t][r];
    };
    if (vec_ok && base + S <= n)
        body(std::true_type{});
    else
        body(std::false_type{});
    __syncthreads();

    for (int t = wave; t < n_trials; t += 4) {
        double pot = 0.0;
#pragma unroll
        for (int r = 0; r < SPT; ++r) {
            const int sl = r * 64 + lane;
            const int64_t i = base + sl;
            if (i < n) {
                const T dist = LITERAL ? part[0][t][sl]
                                       : ((part[0][t][sl] + part[1][t][sl]) + part[2][t][sl]) + part[3][t][sl];
                T v = dist * w_fin[r];
                if (!INIT) v = fmin(v, cl_fin[r]);
                rows[(size_t)t * n + i] = v;
                pot += (double)v;
            }
        }
        const double ws = kmx_wave_sum<double>(pot);
        if (lane == 0) block_pot[(size_t)blockIdx.x * TN_MAX + t] = ws;
    }
    if (INIT && blockIdx.x == 0) {
        for (int f = threadIdx.x; f < d; f += 256) centers_t[(size_t)f * k] = X_t[(size_t)f * n + start];
        if (threadIdx.x == 0) {
            center_indices[0] = start;
            header->best_row = 0;
            header->total = 0.0;
        }
    }
}

// Block-wide exclusive scan of one double per thread (256 threads); returns the exclusive
// prefix of the calling thread and the block total.
__device__ __forceinline__ double block_exclusive_scan(double v, double* wave_tot, double& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    double incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const double o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
    }
    __syncthreads();
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    double base = 0.0;
    for (int w2 = 0; w2 < wave; ++w2) base += wave_tot[w2];
    total = wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
    return base + incl - v;
}

__device__ __forceinline__ int64_t block_min_i64(int64_t v, int64_t* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const int64_t o = __shfl_xor(v, off, 64);
        v = o < v ? o : v;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
    __syncthreads();
    int64_t m = scratch[0];
    for (int w2 = 1; w2 < 4; ++w2) m = scratch[w2] < m ? scratch[w2] : m;
    return m;
}

// One workgroup per trial, plus one that records the selection.
//   do_select: sum the block potentials of every row of the last step, pick the best row
//              (lowest index on ties); the last workgroup records potentials, header and the
//              centre slot and does not sample.
//   do_sample: candidate t = first j with scan(closest)_j >= uniforms[t] * total, and the
//              candidate's feature row for the step kernel.
// Thread i owns the block sums [i * P, (i + 1) * P); with P <= KPP_OWN they are read once and
// stay in registers for the row totals, the coarse scan and the search.
// (KPP_OWN = 4 covers a million samples; 8, for up to 8 trials, two million)
template <typename T, int TN, int KPP_OWN = 4>
__global__ __launch_bounds__(256) void kpp_select_sample_kernel(
    const T* __restrict__ X_t, const double* __restrict__ uniforms,
    const int32_t* __restrict__ cand_prev, int32_t* __restrict__ cand_next,
    int32_t* __restrict__ cand_out, T* __restrict__ centers_t,
    int32_t* __restrict__ center_indices, const T* __restrict__ rows,
    const double* __restrict__ block_pot, double* __restrict__ potentials,
    KppHeader* __restrict__ header, T* __restrict__ cand_rows, int64_t n, int64_t n_blocks, int chunk,
    int d, int k, int n_trials, int center_slot, int do_select, int do_sample) {
    __shared__ double wave_tot[4];
    __shared__ double wave_pot[4][TN];
    __shared__ int64_t iscratch[4];
    __shared__ double prefix_s;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    const int64_t per_thread = (n_blocks + 255) / 256;
    const bool cached = per_thread <= KPP_OWN;
    const int64_t b0 = (int64_t)threadIdx.x * per_thread;
    int64_t b1 = b0 + per_thread;
    if (b1 > n_blocks) b1 = n_blocks;

    int best;
    double own_best[KPP_OWN];  // the owned block sums of the best row (cached mode)
#pragma unroll
    for (int i = 0; i < KPP_OWN; ++i) own_best[i] = 0.0;

    if (do_select) {
        double acc[TN];
        double own[KPP_OWN][TN];
#pragma unroll
        for (int t = 0; t < TN; ++t) acc[t] = 0.0;
        if (cached) {
#pragma unroll
            for (int i = 0; i < KPP_OWN; ++i) {
                const int64_t b = b0 + i;
                const double* __restrict__ rowp = block_pot + (size_t)(b < n_blocks ? b : 0) * TN_MAX;
#pragma unroll
                for (int t = 0; t < TN; ++t) own[i][t] = (b < b1 && t < n_trials) ? rowp[t] : 0.0;
            }
#pragma unroll
            for (int i = 0; i < KPP_OWN; ++i)
#pragma unroll
                for (int t = 0; t < TN; ++t) acc[t] += own[i][t];
        } else {
            for (int64_t b = b0; b < b1; ++b) {
                const double* __restrict__ rowp = block_pot + (size_t)b * TN_MAX;
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    if (t < n_trials) acc[t] += rowp[t];
            }
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            if (t < n_trials) {
                const double ws = kmx_wave_sum<double>(acc[t]);
                if (lane == 0) wave_pot[wave][t] = ws;
            }
        }
        __syncthreads();
        // do_select == 2: the potentials are compared after rounding to T, as the reference's
        // argmin over its T-typed row sums does (kmeans/drivers.py:895-901)
        const bool in_T = do_select == 2;
        double best_pot = (wave_pot[0][0] + wave_pot[1][0]) + (wave_pot[2][0] + wave_pot[3][0]);
        if (in_T) best_pot = (double)(T)best_pot;
        best = 0;
        for (int t = 1; t < n_trials; ++t) {
            double pt = (wave_pot[0][t] + wave_pot[1][t]) + (wave_pot[2][t] + wave_pot[3][t]);
            if (in_T) pt = (double)(T)pt;
            if (pt < best_pot) {
                best_pot = pt;
                best = t;
            }
        }
        if (cached) {
#pragma unroll
            for (int i = 0; i < KPP_OWN; ++i)
#pragma unroll
                for (int t = 0; t < TN; ++t) own_best[i] = (t == best) ? own[i][t] : own_best[i];
        }
        if (blockIdx.x == gridDim.x - 1) {
            const int32_t chosen = cand_prev[best];
            for (int f = threadIdx.x; f < d; f += 256)
                centers_t[(size_t)f * k + center_slot] = X_t[(size_t)f * n + chosen];
            if (threadIdx.x < n_trials)
                potentials[threadIdx.x] = (wave_pot[0][threadIdx.x] + wave_pot[1][threadIdx.x]) +
                                          (wave_pot[2][threadIdx.x] + wave_pot[3][threadIdx.x]);
            if (threadIdx.x == 0) {
                center_indices[center_slot] = chosen;
                header->best_row = best;
                header->total = best_pot;
            }
            return;
        }
    } else {
        best = header->best_row;
        if (cached) {
#pragma unroll
            for (int i = 0; i < KPP_OWN; ++i)
                if (b0 + i < b1) own_best[i] = block_pot[(size_t)(b0 + i) * TN_MAX + best];
        }
    }
    if (!do_sample) return;

    const int trial = blockIdx.x;
    // ---- coarse level: exclusive scan of the block sums of the best row
    double local = 0.0;
    if (cached) {
#pragma unroll
        for (int i = 0; i < KPP_OWN; ++i) local += own_best[i];
    } else {
        for (int64_t b = b0; b < b1; ++b) local += block_pot[(size_t)b * TN_MAX + best];
    }
    double total;
    const double excl = block_exclusive_scan(local, wave_tot, total);
    const double rv = uniforms[trial] * total;
    int64_t found = INT64_MAX;
    double cum = excl, found_prefix = 0.0;
    if (cached) {
#pragma unroll
        for (int i = 0; i < KPP_OWN; ++i) {
            const double before = cum;
            cum += own_best[i];
            if (found == INT64_MAX && b0 + i < b1 && cum >= rv) {
                found = b0 + i;
                found_prefix = before;
            }
        }
    } else {
        for (int64_t b = b0; b < b1; ++b) {
            const double before = cum;
            cum += block_pot[(size_t)b * TN_MAX + best];
            if (cum >= rv) {
                found = b;
                found_prefix = before;
                break;
            }
        }
    }
    const int64_t bstar_raw = block_min_i64(found, iscratch);
    const int64_t bstar = bstar_raw == INT64_MAX ? n_blocks - 1 : bstar_raw;
    if (found == bstar_raw && found != INT64_MAX) prefix_s = found_prefix;
    if (bstar_raw == INT64_MAX && threadIdx.x == 0) prefix_s = total;  // rounding: rv above every cum
    __syncthreads();
    const double prefix = prefix_s;

    // ---- fine level: scan the samples of block bstar (chunk: a multiple of 4, at most 1024)
    const T* __restrict__ closest = rows + (size_t)best * n;
    const int64_t j0 = bstar * chunk + threadIdx.x * 4;
    const bool in_block = (int)threadIdx.x * 4 < chunk;
    double v[4], s = 0.0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        v[r] = (in_block && j0 + r < n) ? (double)closest[j0 + r] : 0.0;
        s += v[r];
    }
    double tot2;
    double c2 = prefix + block_exclusive_scan(s, wave_tot, tot2);
    int64_t hit = INT64_MAX;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        c2 += v[r];
        if (hit == INT64_MAX && in_block && j0 + r < n && c2 >= rv) hit = j0 + r;
    }
    int64_t cand = block_min_i64(hit, iscratch);
    if (cand == INT64_MAX) {
        cand = (bstar + 1) * chunk;  // rounding pushed the crossing just past this block
    }
    if (cand > n - 1) cand = n - 1;
    if (threadIdx.x == 0) {
        cand_next[trial] = (int32_t)cand;
        if (cand_out) cand_out[trial] = (int32_t)cand;
    }
    // the candidate's feature row, for the step kernel
    for (int f = threadIdx.x; f < d; f += 256) cand_rows[(size_t)trial * d + f] = X_t[(size_t)f * n + cand];
}

// The reference's sampler taken literally (kmeans/kernels/kmeans_plusplus.py:79-100): a
// running sum of `closest` in T, element by element from sample 0, and per trial the first j
// whose running sum reaches rv_t = T(u_t) * T(total), clipped to n - 1.  A floating-point
// running sum cannot be split over threads without changing its roundings, so one wave walks the
// array once for all trials (sorted by rv: the sum of non-negative terms never decreases, so
// the trials are met in that order) while the workgroup's 256 threads keep the next 1 024
// values on their way into LDS.  A trial with rv <= 0 leaves the reference's loop at once with
// candidate -1, which its next kernel uses as an index from the end: sample n - 1.
// About 8 ns per sample (8 ms per centre on 10^6 samples): a parity mode, not the default.
template <typename T>
__global__ __launch_bounds__(256) void kpp_sample_literal_kernel(
    const T* __restrict__ X_t, const double* __restrict__ uniforms, int32_t* __restrict__ cand_next,
    int32_t* __restrict__ cand_out, const T* __restrict__ rows, const double* __restrict__ block_pot,
    const KppHeader* __restrict__ header, T* __restrict__ cand_rows, int64_t n, int64_t n_blocks, int d,
    int n_trials) {
    __shared__ T buf[2][CHUNK];
    __shared__ double wave_tot[4];
    __shared__ T rv_sorted[TN_MAX + 1];
    __shared__ int trial_sorted[TN_MAX];
    __shared__ int cand_s[TN_MAX];
    __shared__ int done_s;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int best = header->best_row;
    const T* __restrict__ closest = rows + (size_t)best * n;

    // total potential: the block sums of the best row in fp64, rounded to T once
    double local = 0.0;
    for (int64_t b = threadIdx.x; b < n_blocks; b += 256) local += block_pot[(size_t)b * TN_MAX + best];
    const double ws = kmx_wave_sum<double>(local);
    if (lane == 0) wave_tot[wave] = ws;
    __syncthreads();
    const T total = (T)((wave_tot[0] + wave_tot[1]) + (wave_tot[2] + wave_tot[3]));

    if (threadIdx.x == 0) {
        // insertion sort of the trials by rv; rv <= 0 (or NaN) first
        int m = 0;
        for (int t = 0; t < n_trials; ++t) {
            const T rv = (T)uniforms[t] * total;
            const bool low = !(rv > T(0));
            int pos = m;
            while (pos > 0) {
                const T prev = rv_sorted[pos - 1];
                const bool prev_low = !(prev > T(0));
                if (prev_low || (!low && !(rv < prev))) break;
                rv_sorted[pos] = prev;
                trial_sorted[pos] = trial_sorted[pos - 1];
                --pos;
            }
            rv_sorted[pos] = rv;
            trial_sorted[pos] = t;
            ++m;
        }
        rv_sorted[n_trials] = T(0);
        done_s = 0;
    }
    const int64_t n_chunks = (n + CHUNK - 1) / CHUNK;  // the walk's own chunks, not the block sums
    // first chunk
    {
        const int64_t j0 = (int64_t)threadIdx.x * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) buf[0][threadIdx.x * 4 + r] = (j0 + r < n) ? closest[j0 + r] : T(0);
    }
    __syncthreads();

    int cur = 0;
    T cum = T(0);
    if (wave == 0) {
        // trials that never enter the loop
        while (cur < n_trials && !(rv_sorted[cur] > T(0))) {
            if (lane == 0) cand_s[trial_sorted[cur]] = (int)(n - 1);
            ++cur;
        }
    }
    for (int64_t c = 0; c < n_chunks; ++c) {
        T nxt[4] = {T(0), T(0), T(0), T(0)};
        if (c + 1 < n_chunks) {
            const int64_t j0 = (c + 1) * CHUNK + (int64_t)threadIdx.x * 4;
#pragma unroll
            for (int r = 0; r < 4; ++r) nxt[r] = (j0 + r < n) ? closest[j0 + r] : T(0);
        }
        if (wave == 0) {
            const T* __restrict__ b = buf[c & 1];
            const int64_t base = c * CHUNK;
            const int lim = (int)((n - base) < CHUNK ? (n - base) : CHUNK);
            T rv_cur = rv_sorted[cur];
            for (int i = 0; i < lim && cur < n_trials; i += 16) {
                if (i + 16 <= lim) {
                    T v[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) v[r] = b[i + r];
                    T cc = cum;
#pragma unroll
                    for (int r = 0; r < 16; ++r) cc = cc + v[r];
                    if (rv_cur > cc) {
                        cum = cc;
                        continue;
                    }
                }
                for (int r = 0; r < 16 && i + r < lim; ++r) {
                    cum = cum + b[i + r];
                    while (cur < n_trials && !(rv_cur > cum)) {
                        if (lane == 0) cand_s[trial_sorted[cur]] = (int)(base + i + r);
                        ++cur;
                        rv_cur = rv_sorted[cur];
                    }
                }
            }
            if (lane == 0 && cur >= n_trials) done_s = 1;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) buf[(c + 1) & 1][threadIdx.x * 4 + r] = nxt[r];
        __syncthreads();
        if (done_s) break;
    }
    if (wave == 0 && lane == 0) {
        // the running sum never reached these: the reference's loop stops at the last sample
        for (; cur < n_trials; ++cur) cand_s[trial_sorted[cur]] = (int)(n - 1);
    }
    __syncthreads();
    if (threadIdx.x < n_trials) {
        cand_next[threadIdx.x] = cand_s[threadIdx.x];
        if (cand_out) cand_out[threadIdx.x] = cand_s[threadIdx.x];
    }
    for (int t = 0; t < n_trials; ++t) {
        const int64_t cand = cand_s[t];
        for (int f = threadIdx.x; f < d; f += 256) cand_rows[(size_t)t * d + f] = X_t[(size_t)f * n + cand];
    }
}

struct KppPtrs {
    KppHeader* header;
    void* cand_rows;
    int32_t* cand;
    double* potentials;
    double* block_pot;
    void* rows;
};

KppPtrs kpp_ptrs(char* ws, const KppLayout& L) {
    KppPtrs p;
    p.header = (KppHeader*)(ws + L.off_header);
    p.cand = (int32_t*)(ws + L.off_cand);
    p.cand_rows = ws + L.off_cand_rows;
    p.potentials = (double*)(ws + L.off_pot);
    p.block_pot = (double*)(ws + L.off_block_pot);
    p.rows = ws + L.off_rows;
    return p;
}

int32_t kpp_check(const void* X_t, const void* w, void* ws, size_t ws_bytes, int64_t n, int d, int k,
                  int n_trials, int dtype) {
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(w);
    KMX_REQUIRE_PTR(ws);
    if (n <= 0 || d <= 0 || k <= 0 || n > INT32_MAX) return KMX_ERR_BAD_SHAPE;
    if (n_trials <= 0 || n_trials > TN_MAX) return KMX_ERR_UNSUPPORTED;
    KMX_REQUIRE_DTYPE(dtype);
    if (ws_bytes < kpp_layout(n, d, n_trials, dtype).total) return KMX_ERR_WORKSPACE;
    return KMX_OK;
}

template <typename T>
void launch_init(const void* X_t, const void* w, int32_t start, void* centers_t, int32_t* idx,
                 const KppPtrs& p, const KppLayout& L, int64_t n, int d, int k, hipStream_t s, bool literal) {
    if (L.split) {
        const int vec_ok = (n % L.split == 0) && (((uintptr_t)X_t) % 16 == 0);
#define KMX_KPP_INIT_SPLIT_(SPT, LIT)                                                                 \
    hipLaunchKernelGGL((kpp_step_split_kernel<T, 1, SPT, true, LIT>), dim3((unsigned)L.n_blocks),    \
                       dim3(256), 0, s, (const T*)X_t, (const T*)w, (const T*)nullptr, (T*)p.rows,    \
                       p.block_pot, p.header, n, d, k, 1, vec_ok, start, (T*)centers_t, idx)
#define KMX_KPP_INIT_SPLIT(SPT) \
    do { if (literal) KMX_KPP_INIT_SPLIT_(SPT, true); else KMX_KPP_INIT_SPLIT_(SPT, false); } while (0)
        if (L.split == 1) KMX_KPP_INIT_SPLIT(1);
        else if (L.split == 2) KMX_KPP_INIT_SPLIT(2);
        else if constexpr (sizeof(T) == 4) KMX_KPP_INIT_SPLIT(4);  // (kpp_split: fp32 only)
#undef KMX_KPP_INIT_SPLIT_
#undef KMX_KPP_INIT_SPLIT
        return;
    }
    const int vec_ok = (n % 4 == 0) && (((uintptr_t)X_t) % 16 == 0) && (((uintptr_t)w) % 16 == 0) &&
                       (((uintptr_t)p.rows) % 16 == 0);
#define KMX_KPP_INIT(FUSED)                                                                          \
    hipLaunchKernelGGL((kpp_step_kernel<T, 1, FUSED, true>), dim3((unsigned)L.n_blocks), dim3(256), 0, s, \
                       (const T*)X_t, (const T*)w, (const T*)nullptr, (T*)p.rows, p.block_pot, p.header, \
                       n, d, k, 1, vec_ok, start, (T*)centers_t, idx)
    if (literal) KMX_KPP_INIT(false); else KMX_KPP_INIT(true);
#undef KMX_KPP_INIT
}

template <typename T>
void launch_step(const void* X_t, const void* w, const int32_t* cand, const KppPtrs& p,
                 const KppLayout& L, int64_t n, int d, int n_trials, hipStream_t s, bool literal) {
    (void)cand;  // the candidates' rows were copied to p.cand_rows when they were sampled
    if (L.split) {
        const int vec_split = (n % L.split == 0) && (((uintptr_t)X_t) % 16 == 0);
#define KMX_KPP_STEP_SPLIT_(TN, SPT, LIT)                                                              \
    hipLaunchKernelGGL((kpp_step_split_kernel<T, TN, SPT, false, LIT>), dim3((unsigned)L.n_blocks),    \
                       dim3(256), 0, s, (const T*)X_t, (const T*)w, (const T*)p.cand_rows, (T*)p.rows, \
                       p.block_pot, p.header, n, d, 0, n_trials, vec_split, 0, (T*)nullptr,            \
                       (int32_t*)nullptr)
#define KMX_KPP_STEP_SPLIT(TN, SPT) \
    do { if (literal) KMX_KPP_STEP_SPLIT_(TN, SPT, true); else KMX_KPP_STEP_SPLIT_(TN, SPT, false); } while (0)
        // (which of these exist is kpp_split's choice: the workgroup's partial distances within 32 KB)
        if (n_trials <= 8) {
            if (L.split == 1) KMX_KPP_STEP_SPLIT(8, 1);
            else if (L.split == 2) KMX_KPP_STEP_SPLIT(8, 2);
            else if constexpr (sizeof(T) == 4) KMX_KPP_STEP_SPLIT(8, 4);
        } else {
            if (L.split == 1) KMX_KPP_STEP_SPLIT(TN_MAX, 1);
            else if constexpr (sizeof(T) == 4) KMX_KPP_STEP_SPLIT(TN_MAX, 2);
        }
#undef KMX_KPP_STEP_SPLIT
#undef KMX_KPP_STEP_SPLIT_
        return;
    }
    const int vec_ok = (n % 4 == 0) && (((uintptr_t)X_t) % 16 == 0) && (((uintptr_t)w) % 16 == 0) &&
                       (((uintptr_t)p.rows) % 16 == 0);
#define KMX_KPP_STEP(TN, FUSED)                                                                      \
    hipLaunchKernelGGL((kpp_step_kernel<T, TN, FUSED, false>), dim3((unsigned)L.n_blocks), dim3(256), 0, s, \
                       (const T*)X_t, (const T*)w, (const T*)p.cand_rows, (T*)p.rows, p.block_pot,   \
                       p.header, n, d, 0, n_trials, vec_ok, 0, (T*)nullptr, (int32_t*)nullptr)
    if (n_trials <= 8) {
        if (literal) KMX_KPP_STEP(8, false); else KMX_KPP_STEP(8, true);
    } else {
        if (literal) KMX_KPP_STEP(TN_MAX, false); else KMX_KPP_STEP(TN_MAX, true);
    }
#undef KMX_KPP_STEP
}

template <typename T>
void launch_select_sample(const void* X_t, const double* uniforms, const int32_t* cand_prev,
                          int32_t* cand_next, int32_t* cand_out, void* centers_t, int32_t* idx,
                          const KppPtrs& p, const KppLayout& L, int64_t n, int d, int k,
                          int n_trials, int slot, int do_select, int do_sample, hipStream_t s,
                          bool literal = false) {
    if (literal) {
        // the selection alone (potentials compared in T), then the serial walk of one workgroup
        if (do_select)
            launch_select_sample<T>(X_t, uniforms, cand_prev, cand_next, cand_out, centers_t, idx, p, L, n, d, k,
                                    n_trials, slot, 2, 0, s);
        if (do_sample)
            hipLaunchKernelGGL((kpp_sample_literal_kernel<T>), dim3(1), dim3(256), 0, s, (const T*)X_t, uniforms,
                               cand_next, cand_out, (const T*)p.rows, p.block_pot, p.header, (T*)p.cand_rows, n,
                               L.n_blocks, d, n_trials);
        return;
    }
    // one workgroup per trial when sampling, one more when a selection is recorded
    const unsigned grid = (do_sample ? (unsigned)n_trials : 0u) + (do_select ? 1u : 0u);
    if (grid == 0) return;
#define KMX_KPP_SELECT(...)                                                                       \
    hipLaunchKernelGGL((kpp_select_sample_kernel<T, __VA_ARGS__>), dim3(grid), dim3(256), 0, s,    \
                       (const T*)X_t, uniforms, cand_prev, cand_next, cand_out, (T*)centers_t, idx, \
                       (const T*)p.rows, p.block_pot, p.potentials, p.header, (T*)p.cand_rows, n,   \
                       L.n_blocks, L.chunk, d, k, n_trials, slot, do_select, do_sample)
    if (n_trials <= 8) {
        // (more than four block sums per thread: eight in registers rather than re-read)
        if (L.n_blocks > 4 * 256 && L.n_blocks <= 8 * 256) KMX_KPP_SELECT(8, 8);
        else KMX_KPP_SELECT(8);
    } else {
        KMX_KPP_SELECT(TN_MAX);
    }
#undef KMX_KPP_SELECT
}

}  // namespace

extern "C" {

size_t kmx_kpp_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype) {
    (void)k;
    if (n <= 0 || n_trials <= 0 || n_trials > TN_MAX || (dtype != KMX_F32 && dtype != KMX_F64))
        return 0;
    return kpp_layout(n, d, n_trials, dtype).total;
}

int32_t kmx_kpp_init(const void* X_t, const void* sample_weight, int32_t start_index,
                     void* centers_t, int32_t* center_indices, void* workspace,
                     size_t workspace_bytes, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                     int32_t dtype, uint32_t flags, void* stream_) {
    KMX_ENTRY();
    const int32_t rc = kpp_check(X_t, sample_weight, workspace, workspace_bytes, n, d, k, n_trials, dtype);
    if (rc != KMX_OK) return rc;
    KMX_REQUIRE_PTR(centers_t);
    KMX_REQUIRE_PTR(center_indices);
    if (flags & ~(uint32_t)KMX_KPP_SAMPLER_LITERAL) return KMX_ERR_BAD_ARGUMENT;
    const bool literal = (flags & KMX_KPP_SAMPLER_LITERAL) != 0;
    if (start_index < 0 || start_index >= n) return KMX_ERR_BAD_ARGUMENT;
    const KppLayout L = kpp_layout(n, d, n_trials, dtype);
    const KppPtrs p = kpp_ptrs((char*)workspace, L);
    hipStream_t s = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        launch_init<float>(X_t, sample_weight, start_index, centers_t, center_indices, p, L, n, d, k, s, literal);
    else
        launch_init<double>(X_t, sample_weight, start_index, centers_t, center_indices, p, L, n, d, k, s, literal);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_kpp_sample_candidates(const void* X_t, const double* uniforms_for_step,
                                  int32_t* candidates, void* workspace, size_t workspace_bytes,
                                  int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype,
                                  uint32_t flags, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(uniforms_for_step);
    if (flags & ~(uint32_t)KMX_KPP_SAMPLER_LITERAL) return KMX_ERR_BAD_ARGUMENT;
    const bool literal = (flags & KMX_KPP_SAMPLER_LITERAL) != 0;
    const int32_t rc = kpp_check(X_t, uniforms_for_step, workspace, workspace_bytes, n, d, k, n_trials, dtype);
    if (rc != KMX_OK) return rc;
    const KppLayout L = kpp_layout(n, d, n_trials, dtype);
    const KppPtrs p = kpp_ptrs((char*)workspace, L);
    hipStream_t s = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        launch_select_sample<float>(X_t, uniforms_for_step, p.cand, p.cand, candidates, nullptr,
                                    nullptr, p, L, n, d, k, n_trials, 0, 0, 1, s, literal);
    else
        launch_select_sample<double>(X_t, uniforms_for_step, p.cand, p.cand, candidates, nullptr,
                                     nullptr, p, L, n, d, k, n_trials, 0, 0, 1, s, literal);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_kpp_step(const void* X_t, const void* sample_weight, int32_t center_slot,
                     void* centers_t, int32_t* center_indices, void* workspace,
                     size_t workspace_bytes, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                     int32_t dtype, uint32_t flags, void* stream_) {
    KMX_ENTRY();
    const int32_t rc = kpp_check(X_t, sample_weight, workspace, workspace_bytes, n, d, k, n_trials, dtype);
    if (rc != KMX_OK) return rc;
    KMX_REQUIRE_PTR(centers_t);
    KMX_REQUIRE_PTR(center_indices);
    if (flags & ~(uint32_t)KMX_KPP_SAMPLER_LITERAL) return KMX_ERR_BAD_ARGUMENT;
    const bool literal = (flags & KMX_KPP_SAMPLER_LITERAL) != 0;
    if (center_slot < 1 || center_slot >= k) return KMX_ERR_BAD_ARGUMENT;
    const KppLayout L = kpp_layout(n, d, n_trials, dtype);
    const KppPtrs p = kpp_ptrs((char*)workspace, L);
    hipStream_t s = (hipStream_t)stream_;
    if (dtype == KMX_F32) {
        launch_step<float>(X_t, sample_weight, p.cand, p, L, n, d, n_trials, s, literal);
        launch_select_sample<float>(X_t, nullptr, p.cand, nullptr, nullptr, centers_t, center_indices,
                                    p, L, n, d, k, n_trials, center_slot, 1, 0, s, literal);
    } else {
        launch_step<double>(X_t, sample_weight, p.cand, p, L, n, d, n_trials, s, literal);
        launch_select_sample<double>(X_t, nullptr, p.cand, nullptr, nullptr, centers_t,
                                     center_indices, p, L, n, d, k, n_trials, center_slot, 1, 0, s, literal);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_kpp_run(const void* X_t, const void* sample_weight, const double* uniforms,
                    int32_t start_index, void* centers_t, int32_t* center_indices,
                    void* workspace, size_t workspace_bytes, int64_t n, int32_t d, int32_t k,
                    int32_t n_trials, int32_t dtype, uint32_t flags, void* stream_) {
    KMX_ENTRY();
    if (flags & ~(uint32_t)KMX_KPP_SAMPLER_LITERAL) return KMX_ERR_BAD_ARGUMENT;
    const bool literal = (flags & KMX_KPP_SAMPLER_LITERAL) != 0;
    int32_t rc = kmx_kpp_init(X_t, sample_weight, start_index, centers_t, center_indices, workspace,
                              workspace_bytes, n, d, k, n_trials, dtype, flags, stream_);
    if (rc != KMX_OK) return rc;
    if (k == 1) return KMX_OK;
    KMX_REQUIRE_PTR(uniforms);
    const KppLayout L = kpp_layout(n, d, n_trials, dtype);
    const KppPtrs p = kpp_ptrs((char*)workspace, L);
    hipStream_t s = (hipStream_t)stream_;
    for (int c = 1; c < k; ++c) {
        // candidates alternate between two buffers: the fused launch reads the previous
        // step's candidates (to record its winner) while it writes the next ones
        int32_t* cand_prev = p.cand + ((c - 1) & 1) * TN_MAX;
        int32_t* cand_next = p.cand + (c & 1) * TN_MAX;
        const double* u = uniforms + (size_t)(c - 1) * n_trials;
        const int do_select = c > 1 ? 1 : 0;
        if (dtype == KMX_F32) {
            launch_select_sample<float>(X_t, u, cand_prev, cand_next, nullptr, centers_t,
                                        center_indices, p, L, n, d, k, n_trials, c - 1, do_select, 1, s, literal);
            launch_step<float>(X_t, sample_weight, cand_next, p, L, n, d, n_trials, s, literal);
        } else {
            launch_select_sample<double>(X_t, u, cand_prev, cand_next, nullptr, centers_t,
                                         center_indices, p, L, n, d, k, n_trials, c - 1, do_select, 1, s, literal);
            launch_step<double>(X_t, sample_weight, cand_next, p, L, n, d, n_trials, s, literal);
        }
        KMX_LAUNCH_CHECK();
    }
    int32_t* cand_last = p.cand + ((k - 1) & 1) * TN_MAX;
    if (dtype == KMX_F32)
        launch_select_sample<float>(X_t, nullptr, cand_last, nullptr, nullptr, centers_t,
                                    center_indices, p, L, n, d, k, n_trials, k - 1, 1, 0, s, literal);
    else
        launch_select_sample<double>(X_t, nullptr, cand_last, nullptr, nullptr, centers_t,
                                     center_indices, p, L, n, d, k, n_trials, k - 1, 1, 0, s, literal);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

void* kmx_kpp_closest_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                          int32_t dtype) {
    (void)k;
    if (!workspace || n <= 0 || n_trials <= 0) return nullptr;
    // start of the rows; the caller adds best_row * n elements (best_row from the header)
    return (char*)workspace + kpp_layout(n, d, n_trials, dtype).off_rows;
}

double* kmx_kpp_potentials_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                               int32_t dtype) {
    (void)k;
    if (!workspace || n <= 0 || n_trials <= 0) return nullptr;
    return (double*)((char*)workspace + kpp_layout(n, d, n_trials, dtype).off_pot);
}

int32_t* kmx_kpp_candidates_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                                int32_t dtype) {
    (void)k;
    if (!workspace || n <= 0 || n_trials <= 0) return nullptr;
    return (int32_t*)((char*)workspace + kpp_layout(n, d, n_trials, dtype).off_cand);
}

}  // extern "C"
