// Single-workgroup finalisation of a Lloyd iteration, used when (d + 1) * k is small enough
// for one workgroup: empty-cluster list (ascending) and heaviest cluster, then division by
// the cluster sizes, packed centroid copy and half squared norms for the next iteration,
// centroid shift and the convergence test.  Every sum is taken in a fixed order.
#pragma once

#include "kmx_common.h"

template <typename T>
struct LloydTail {
    T* sums_t;               // (d, k): sums on entry, the new centroids on exit
    T* sizes;                // OUT (k)
    uint32_t* empty_clusters;
    const T* old_centroids_t;
    T* cpack;
    T* half_norms;
    kmx_lloyd_status* status;
    int d, k, dpad;
    uint32_t* clear_word = nullptr;  // a counter to copy to the next word and zero, or null
    // Screened fused step only: word clear_word[2] tells the next step whether it may correct the
    // fixed-point sums for the samples that change cluster instead of rebuilding them; the sums
    // then stay in `gsum` instead of being cleared.  Chosen when the iteration just finished
    // changed at most n_samples / delta_divisor labels (0: always rebuild): the word is then 2,
    // or 1 when it changed at most n_samples / list_divisor labels (few enough for the step to
    // collect them in a list and deal with them after its last tile).
    int64_t n_samples = 0;
    int delta_divisor = 0;
    int list_divisor = 0;
};

// Empty-cluster list (ascending) and heaviest cluster; one workgroup of up to 1024 threads, all
// of which call it.  Returns the number of empty clusters (same value in every thread).
template <typename T>
__device__ inline int lloyd_list_empty(const T* sizes, uint32_t* empty_clusters, int k,
                                       int* heaviest_out) {
    __shared__ int wave_counts[16];
    __shared__ T hv_val[16];
    __shared__ int hv_idx[16];
    __shared__ int result_s[2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_threads = (int)blockDim.x, n_waves = (n_threads + 63) >> 6;
    int base = 0;
    T my_max = -kmx_inf<T>();
    int my_arg = 0x7fffffff;
    for (int c0 = 0; c0 < k; c0 += n_threads) {
        const int c = c0 + threadIdx.x;
        T sz = T(1);
        if (c < k) {
            sz = sizes[c];
            if (sz > my_max) {
                my_max = sz;
                my_arg = c;
            }
        }
        const bool flag = (c < k) && (sz == T(0));
        const unsigned long long mask = __ballot(flag);
        const int prefix = __popcll(mask & ((1ull << lane) - 1ull));
        __syncthreads();
        if (lane == 0) wave_counts[wave] = __popcll(mask);
        __syncthreads();
        int offset = base;
        for (int w2 = 0; w2 < wave; ++w2) offset += wave_counts[w2];
        if (flag) empty_clusters[offset + prefix] = (uint32_t)c;
        for (int w2 = 0; w2 < n_waves; ++w2) base += wave_counts[w2];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const T ov = __shfl_xor(my_max, off, 64);
        const int oi = __shfl_xor(my_arg, off, 64);
        if (ov > my_max || (ov == my_max && oi < my_arg)) {
            my_max = ov;
            my_arg = oi;
        }
    }
    __syncthreads();
    if (lane == 0) {
        hv_val[wave] = my_max;
        hv_idx[wave] = my_arg;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        T bv = hv_val[0];
        int bidx = hv_idx[0];
        for (int w2 = 1; w2 < n_waves; ++w2) {
            if (hv_val[w2] > bv || (hv_val[w2] == bv && hv_idx[w2] < bidx)) {
                bv = hv_val[w2];
                bidx = hv_idx[w2];
            }
        }
        result_s[0] = bidx;
    }
    __syncthreads();
    *heaviest_out = result_s[0];
    return base;
}

// The same for at most 64 clusters, by the first wave alone and with one barrier (the general
// routine above passes five, each a wait for all the waves of the workgroup).
template <typename T>
__device__ inline int lloyd_list_empty_one_wave(const T* sizes, uint32_t* empty_clusters, int k,
                                                int* heaviest_out) {
    __shared__ int one_wave_result[2];
    if (threadIdx.x < 64) {
        const int c = (int)threadIdx.x;
        const bool in = c < k;
        const T sz = in ? sizes[c] : T(1);
        const bool flag = in && sz == T(0);
        const unsigned long long mask = __ballot(flag);
        if (flag) empty_clusters[__popcll(mask & ((1ull << c) - 1ull))] = (uint32_t)c;
        T my_max = in ? sz : -kmx_inf<T>();
        int my_arg = in ? c : 0x7fffffff;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const T ov = __shfl_xor(my_max, off, 64);
            const int oi = __shfl_xor(my_arg, off, 64);
            if (ov > my_max || (ov == my_max && oi < my_arg)) {
                my_max = ov;
                my_arg = oi;
            }
        }
        if (c == 0) {
            one_wave_result[0] = my_arg;
            one_wave_result[1] = __popcll(mask);
        }
    }
    __syncthreads();
    *heaviest_out = one_wave_result[0];
    return one_wave_result[1];
}

// End of an iteration, by one thread: iteration count, shift, and the next state (strict
// convergence from the second iteration on, then the tolerance, then the iteration limit).
__device__ inline void lloyd_update_status(kmx_lloyd_status* st, double total_shift, unsigned int changed) {
    const int n_iter = st->n_iter + 1;
    st->n_iter = n_iter;
    st->shift_sum = total_shift;
    st->n_changed = 0;
    int next = KMX_RUNNING;
    if (n_iter > 1 && changed == 0)
        next = KMX_CONVERGED_STRICT;
    else if (!(total_shift > st->tol))
        next = KMX_CONVERGED_TOL;
    else if (n_iter >= st->max_iter)
        next = KMX_MAX_ITER;
    st->state = next;
    st->reserved[1] = (int64_t)changed;
}

// Division, packed copy, half norms, shift and convergence test by ONE workgroup of 256
// threads (thread per cluster, features in order).  `sums_t` becomes the new centroids.
template <typename T>
__device__ inline void lloyd_finalize_block(const LloydTail<T>& a, int n_empty, int heaviest) {
    __shared__ double scratch[4];
    const int d = a.d, k = a.k, dpad = a.dpad;
    double shift = 0.0;
    for (int c = threadIdx.x; c < k; c += 256) {
        const T sz = a.sizes[c];
        if (sz != T(0)) {
            T sq = T(0), sh = T(0);
#pragma unroll 2
            for (int f = 0; f < d; ++f) {
                const T nv = a.sums_t[(size_t)f * k + c] / sz;
                const T df = a.old_centroids_t[(size_t)f * k + c] - nv;
                sh += df * df;
                sq += nv * nv;
                a.cpack[(size_t)c * dpad + f] = nv;
                a.sums_t[(size_t)f * k + c] = nv;
            }
            for (int f = d; f < dpad; ++f) a.cpack[(size_t)c * dpad + f] = T(0);
            a.half_norms[c] = sq / T(2);
            shift += (double)sh;
        }
    }
    __syncthreads();
    if (n_empty > 0) {
        // still-empty clusters (nothing could be relocated) are parked on the heaviest one
        for (int c = threadIdx.x; c < k; c += 256) {
            if (a.sizes[c] == T(0)) {
                T sq = T(0), sh = T(0);
                for (int f = 0; f < d; ++f) {
                    const T nv = a.cpack[(size_t)heaviest * dpad + f];
                    const T df = a.old_centroids_t[(size_t)f * k + c] - nv;
                    sh += df * df;
                    sq += nv * nv;
                    a.cpack[(size_t)c * dpad + f] = nv;
                    a.sums_t[(size_t)f * k + c] = nv;
                }
                for (int f = d; f < dpad; ++f) a.cpack[(size_t)c * dpad + f] = T(0);
                a.half_norms[c] = sq / T(2);
                shift += (double)sh;
            }
        }
    }
    const double total = kmx_block_sum<double>(shift, scratch);
    if (threadIdx.x == 0) lloyd_update_status(a.status, total, a.status->n_changed);
}


// One workgroup (every thread of it, up to 1024) finishes an iteration whose (d + 1) * k sums fit
// in LDS: empty-cluster list and, if no cluster is empty, division by the sizes, packed copy and
// half norms for the next iteration, centroid shift, convergence test.  The sums stay in LDS
// (`vals`, (d + 1) * k elements) between the phases; global memory is read once and written once
// per output.
//   FROM_GSUM: the sums arrive as 64-bit fixed point (`gsum`, binary point q_exp[f]) and are
//              converted, stored to sums_t / sizes and cleared here;
//   otherwise: sums_t / sizes already hold the reduced sums.
// With an empty cluster the raw sums and sizes stay in global memory for the relocation and
// the state becomes KMX_NEED_RELOCATION.
//   COHERENT: called by the last workgroup of the launch whose workgroups produced the sums, the
//             changed-label count and the counter word with device-scope atomics (and waited for
//             them before they drew their ticket): those words are read with device-scope loads,
//             which do not stop at a cache of the own chiplet that may hold an older copy.
//   WIDE: hundreds of features and few clusters, at most as many as threads (takes 4 KB of LDS
//         more: a cluster's norm by a group of threads).
template <typename T, bool FROM_GSUM, bool COHERENT, bool WIDE = false>
__device__ inline void lloyd_small_finalize_body(unsigned long long* __restrict__ gsum,
                                                 const int* __restrict__ q_exp, const LloydTail<T>& a,
                                                 T* __restrict__ vals) {
    __shared__ double scratch[16];
    const int n_threads = (int)blockDim.x;
    // Element jx = f k + c of the (d + 1, k) arrays is taken by thread jx % stride in its pass
    // jx / stride.  WIDE: stride is the largest multiple of k within the workgroup, so that a thread
    // keeps its cluster and moves on by stride / k features per pass - with thousands of elements
    // the division of every index by k, three times per element, was most of what this workgroup,
    // alone on its compute unit, had to issue.
    const int rows_per_pass = WIDE ? n_threads / a.k : 0;
    const int stride = WIDE ? rows_per_pass * a.k : n_threads;
    const bool lane_on = (int)threadIdx.x < stride;
    const int f_first = WIDE ? (int)threadIdx.x / a.k : 0;
    const int c_mine = WIDE ? (int)threadIdx.x - f_first * a.k : 0;
    // feature of the element jx that the thread takes in pass `pass`
    auto feature_of = [&](const int jx, const int pass) __attribute__((always_inline)) {
        return WIDE ? f_first + pass * rows_per_pass : jx / a.k;
    };
    // The old centroids are asked for before anything else (up to eight values per thread: what
    // (d + 1) k <= 2048 needs with 256 threads): the routine is a chain of memory round trips, and
    // this one then runs beside those of the state and of the sums ...
    constexpr int OLD_AHEAD = 8;
    const int dk_ahead = a.d * a.k;
    const bool old_ahead = dk_ahead <= stride * OLD_AHEAD;
    T old_v[OLD_AHEAD];
#pragma unroll
    for (int i = 0; i < OLD_AHEAD; ++i) {
        const int jx = (int)threadIdx.x + stride * i;
        old_v[i] = (old_ahead && lane_on && jx < dk_ahead) ? a.old_centroids_t[jx] : T(0);
    }
    const int d = a.d, k = a.k, dpad = a.dpad;
    const int items = (d + 1) * k, dk = d * k;
    // ... and so are the sums themselves (up to eight per thread), the changed-label count and
    // the counter word: one round trip for all of them instead of one after the other
    auto load_sum = [&](const int jx) __attribute__((always_inline)) {
        return (long long)(COHERENT ? __hip_atomic_load(&gsum[jx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                    : gsum[jx]);
    };
    constexpr int SUMS_AHEAD = 8;
    const bool sums_ahead = FROM_GSUM && items <= stride * SUMS_AHEAD;
    long long sum_v[SUMS_AHEAD];
    int q_v[SUMS_AHEAD];  // (their binary points, asked for in the same round trip)
    if constexpr (FROM_GSUM) {
#pragma unroll
        for (int i = 0; i < SUMS_AHEAD; ++i) {
            const int jx = (int)threadIdx.x + stride * i;
            const bool mine = sums_ahead && lane_on && jx < items;
            sum_v[i] = mine ? load_sum(jx) : 0ll;
            q_v[i] = mine ? q_exp[feature_of(jx, i)] : 0;
        }
    }
    unsigned int counter_word = 0u;
    if (a.clear_word != nullptr && threadIdx.x == 0)
        counter_word = COHERENT ? __hip_atomic_load(&a.clear_word[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                : a.clear_word[0];
    const unsigned int n_changed =
        COHERENT ? __hip_atomic_load(&a.status->n_changed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                 : a.status->n_changed;
    if (a.clear_word != nullptr && threadIdx.x == 0) {
        a.clear_word[1] = counter_word;  // kept for kmx_lloyd_recheck_count
        a.clear_word[0] = 0u;
    }
    const T* sizes_s = vals + dk;  // vals: [(d + 1) * k], sums, then sizes
    T* __restrict__ out_t = a.sums_t;
    const T* __restrict__ old_t = a.old_centroids_t;
    // (the label changes of the iteration at hand; every thread reads the same word before
    // thread 0 resets it at the end of the kernel)
    const bool keep_sums = FROM_GSUM && a.clear_word != nullptr && a.delta_divisor > 0 &&
                           (int64_t)n_changed * a.delta_divisor <= a.n_samples;
    // WIDE, with every element already in a register of its thread: the sizes are converted
    // first, and each sum is converted, divided and stored in one go once no cluster is known to be
    // empty
    const bool fused = WIDE && FROM_GSUM && sums_ahead && old_ahead;
    T raw_v[SUMS_AHEAD];
#pragma unroll
    for (int i = 0; i < SUMS_AHEAD; ++i) raw_v[i] = T(0);
    if constexpr (FROM_GSUM) {
        auto convert = [&](const int jx, const int f, const long long iv, const int q) __attribute__((always_inline)) {
            if (!keep_sums) gsum[jx] = 0ull;
            // (times 2^-q, built from its exponent field: exact, like ldexp)
            const T val = (T)((double)iv * __hiloint2double((1023 - q) << 20, 0));
            vals[jx] = val;
            if (f < d)
                out_t[jx] = val;
            else
                a.sizes[jx - dk] = val;
        };
        if (sums_ahead) {
#pragma unroll
            for (int i = 0; i < SUMS_AHEAD; ++i) {
                const int jx = (int)threadIdx.x + stride * i;
                if (lane_on && jx < items) {
                    const int f = feature_of(jx, i);
                    if (fused && f < d) {
                        // (kept in its register until the sizes are known: no store of the raw sum,
                        // no trip through the LDS)
                        if (!keep_sums) gsum[jx] = 0ull;
                        raw_v[i] = (T)((double)sum_v[i] * __hiloint2double((1023 - q_v[i]) << 20, 0));
                    } else {
                        convert(jx, f, sum_v[i], q_v[i]);
                    }
                }
            }
        } else {
            // (SUMS_AHEAD loads in flight per thread and pass: a loop of one load and one store per
            // pass would take a trip to memory per element)
            for (int base = 0, pass0 = 0; base < items; base += stride * SUMS_AHEAD, pass0 += SUMS_AHEAD) {
#pragma unroll
                for (int i = 0; i < SUMS_AHEAD; ++i) {
                    const int jx = base + (int)threadIdx.x + stride * i;
                    const bool mine = lane_on && jx < items;
                    sum_v[i] = mine ? load_sum(jx) : 0ll;
                    q_v[i] = mine ? q_exp[feature_of(jx, pass0 + i)] : 0;
                }
#pragma unroll
                for (int i = 0; i < SUMS_AHEAD; ++i) {
                    const int jx = base + (int)threadIdx.x + stride * i;
                    if (lane_on && jx < items) convert(jx, feature_of(jx, pass0 + i), sum_v[i], q_v[i]);
                }
            }
        }
    } else {
        for (int jx = threadIdx.x; jx < items; jx += n_threads) vals[jx] = jx < dk ? out_t[jx] : a.sizes[jx - dk];
    }
    __syncthreads();
    int heaviest = 0;
    const int n_empty = (WIDE && k <= 64) ? lloyd_list_empty_one_wave<T>(sizes_s, a.empty_clusters, k, &heaviest)
                                          : lloyd_list_empty<T>(sizes_s, a.empty_clusters, k, &heaviest);
    if (threadIdx.x == 0) {
        a.status->n_empty = n_empty;
        a.status->reserved[0] = heaviest;
    }
    if (n_empty > 0) {
        // the host relocates and finishes the iteration; the next step rebuilds the sums
        if constexpr (FROM_GSUM) {
            if (keep_sums)
                for (int jx = threadIdx.x; jx < items; jx += n_threads) gsum[jx] = 0ull;
            if (fused) {  // (the raw sums, as the relocation reads them)
#pragma unroll
                for (int i = 0; i < SUMS_AHEAD; ++i) {
                    const int jx = (int)threadIdx.x + stride * i;
                    if (lane_on && jx < dk) out_t[jx] = raw_v[i];
                }
            }
        }
        if (threadIdx.x == 0) {
            a.status->state = KMX_NEED_RELOCATION;
            if (a.clear_word != nullptr) a.clear_word[2] = 0u;
        }
        return;
    }
    if (a.clear_word != nullptr && threadIdx.x == 0)
        a.clear_word[2] = !keep_sums ? 0u
                          : (a.list_divisor > 0 && (int64_t)n_changed * a.list_divisor <= a.n_samples) ? 1u
                                                                                                    : 2u;
    double shift = 0.0;
    // (a.cpack may be null: the caller's kernels read the (d, k) array only)
    const T size_mine = WIDE ? sizes_s[c_mine] : T(1);
    auto divide = [&](const int jx, const int f, const T old_value, const T raw) __attribute__((always_inline)) {
        const int c = WIDE ? c_mine : jx - f * k;
        const T nv = (fused ? raw : vals[jx]) / (WIDE ? size_mine : sizes_s[c]);
        const T df = old_value - nv;
        shift += (double)(df * df);
        vals[jx] = nv;
        out_t[jx] = nv;
        if (a.cpack != nullptr) a.cpack[(size_t)c * dpad + f] = nv;
    };
    if (old_ahead) {  // (the same elements in the same order as the loop below)
#pragma unroll
        for (int i = 0; i < OLD_AHEAD; ++i) {
            const int jx = (int)threadIdx.x + stride * i;
            if (lane_on && jx < dk) divide(jx, feature_of(jx, i), old_v[i], raw_v[i]);
        }
    } else {
        for (int base = 0, pass0 = 0; base < dk; base += stride * OLD_AHEAD, pass0 += OLD_AHEAD) {
#pragma unroll
            for (int i = 0; i < OLD_AHEAD; ++i) {
                const int jx = base + (int)threadIdx.x + stride * i;
                old_v[i] = (lane_on && jx < dk) ? old_t[jx] : T(0);
            }
#pragma unroll
            for (int i = 0; i < OLD_AHEAD; ++i) {
                const int jx = base + (int)threadIdx.x + stride * i;
                if (lane_on && jx < dk) divide(jx, feature_of(jx, pass0 + i), old_v[i], T(0));
            }
        }
    }
    __syncthreads();
    if constexpr (WIDE) {
        // wide samples, few clusters: a cluster's norm by a group of threads (thread (g, c) takes
        // every n_g-th feature, the groups are then added in order) - one thread per cluster
        // would walk hundreds of features alone while the others wait
        // (the groups are added in two steps - eight threads per cluster take every eighth group,
        // then one adds the eight - where one thread alone would walk a hundred values, a trip to
        // the LDS each)
        __shared__ T norm_part[1024];
        __shared__ T norm_part8[8 * 64];
        const int n_g = n_threads / k;
        const int c = (int)threadIdx.x % k, g = (int)threadIdx.x / k;
        T sq = T(0);
        if (g < n_g)
            for (int f = g; f < d; f += n_g) sq += vals[f * k + c] * vals[f * k + c];
        norm_part[threadIdx.x] = sq;
        __syncthreads();
        const bool two_steps = k <= 64 && n_g >= 16;
        if (two_steps) {
            if (g < 8) {
                T tot = norm_part[g * k + c];
                for (int g2 = g + 8; g2 < n_g; g2 += 8) tot += norm_part[g2 * k + c];
                norm_part8[g * k + c] = tot;
            }
            __syncthreads();
        }
        if ((int)threadIdx.x < k) {
            T tot;
            if (two_steps) {
                tot = norm_part8[threadIdx.x];
                for (int g2 = 1; g2 < 8; ++g2) tot += norm_part8[g2 * k + threadIdx.x];
            } else {
                tot = norm_part[threadIdx.x];
                for (int g2 = 1; g2 < n_g; ++g2) tot += norm_part[g2 * k + threadIdx.x];
            }
            a.half_norms[threadIdx.x] = tot / T(2);
            if (a.cpack != nullptr)
                for (int f = d; f < dpad; ++f) a.cpack[(size_t)threadIdx.x * dpad + f] = T(0);
        }
    } else {
        for (int c = threadIdx.x; c < k; c += n_threads) {
            T sq = T(0);
            for (int f = 0; f < d; ++f) sq += vals[f * k + c] * vals[f * k + c];
            a.half_norms[c] = sq / T(2);
            for (int f = d; f < dpad; ++f) a.cpack[(size_t)c * dpad + f] = T(0);
        }
    }
    const double total = kmx_block_sum<double>(shift, scratch);
    if (threadIdx.x == 0) lloyd_update_status(a.status, total, n_changed);
}

// The same as a launch of its own: ordered after the producers of the sums by the kernel boundary.
template <typename T, bool FROM_GSUM>
__global__ __launch_bounds__(256) void lloyd_small_finalize_kernel(
    unsigned long long* __restrict__ gsum, const int* __restrict__ q_exp, LloydTail<T> a) {
    extern __shared__ __align__(16) unsigned char fin_raw[];
    if (a.status->state != KMX_RUNNING) return;
    lloyd_small_finalize_body<T, FROM_GSUM, false>(gsum, q_exp, a, reinterpret_cast<T*>(fin_raw));
}
