// Lloyd iteration for gfx950: fused assignment + partial centroid sums, reduction of the
// partial sums with empty-cluster detection, and the finalisation (division, shift,
// convergence test).  Public entry points are declared in include/mi355x_kmeans.h.
//
// Fused step, vector-ALU variants (this file):
//   * "register" path: every thread keeps R samples (all features) in registers, read once
//     from X_t with 128-bit loads; centroids come from a packed (k, dpad) copy through
//     wave-uniform (scalar) loads, so the inner loop is one v_fma per (sample, feature,
//     centroid) with the centroid value in an SGPR;
//   * "streaming" path for wide samples: windows of 8 centroids, features re-read per window.
// Partial sums of w*x and w go to LDS accumulators private to the workgroup (flushed once
// per workgroup) when (d + 1) * k values fit, else to a few global copies with hardware
// float atomics.  The MFMA variant for fp32 lives in lloyd_mfma.hip.
#include "kmx_common.h"
#include "lloyd_layout.h"

#include <mutex>
#include <vector>
#include "lloyd_tail.h"

namespace {

template <typename T, int R>
struct VecOf;
template <>
struct VecOf<float, 1> { using type = float; };
template <>
struct VecOf<float, 2> { using type = float2; };
template <>
struct VecOf<float, 4> { using type = float4; };
template <>
struct VecOf<double, 1> { using type = double; };
template <>
struct VecOf<double, 2> { using type = double2; };

// R consecutive samples of one feature row; vector load when the row is aligned.
template <typename T, int R>
__device__ __forceinline__ void load_row(const T* __restrict__ row, int64_t i0, int64_t n,
                                         bool vec_ok, T (&out)[R]) {
    if (vec_ok && i0 + R <= n) {
        using V = typename VecOf<T, R>::type;
        union {
            V v;
            T s[R];
        } u;
        u.v = *reinterpret_cast<const V*>(row + i0);
#pragma unroll
        for (int r = 0; r < R; ++r) out[r] = u.s[r];
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) out[r] = (i0 + r < n) ? row[i0 + r] : T(0);
    }
}

constexpr int ACC_NONE = 0;    // labels only
constexpr int ACC_LDS = 1;     // workgroup-private LDS accumulators, flushed to partial[block]
constexpr int ACC_GLOBAL = 2;  // hardware float atomics into partial[block % n_copies]

// ------------------------------------------------------------------------------------------
// Register-resident fused step.
// ------------------------------------------------------------------------------------------
template <typename T, int DREG, int R, int ACC>
__global__ __launch_bounds__(256) void lloyd_fused_reg_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight, const T* __restrict__ cpack,
    const T* __restrict__ half_norms, const uint32_t* __restrict__ labels_prev,
    uint32_t* __restrict__ labels, T* __restrict__ partial, kmx_lloyd_status* __restrict__ status,
    int64_t n, int d, int k, int dpad, int n_copies, int vec_ok, int lds_copies) {
    if (status != nullptr && status->state != KMX_RUNNING) return;

    // LDS accumulators are fp64 for both types: ds_add_f64 is fast on this hardware, ds_add_f32
    // is not (about 195 cycles per wave instruction)
    extern __shared__ __align__(16) unsigned char smem_raw[];
    double* acc = reinterpret_cast<double*>(smem_raw);
    __shared__ unsigned int changed_block;
    const int items = (d + 1) * k;
    if (ACC == ACC_LDS) {
        for (int j = threadIdx.x; j < items * lds_copies; j += 256) acc[j] = 0.0;
        // few clusters mean many lanes of a wave on one address: lanes spread over copies
        acc += (size_t)(threadIdx.x & (lds_copies - 1)) * items;
    }
    if (threadIdx.x == 0) changed_block = 0;
    __syncthreads();

    T* gacc = (ACC == ACC_GLOBAL) ? partial + (size_t)(blockIdx.x % n_copies) * items : nullptr;
    unsigned int changed = 0;
    const int64_t tile_samples = 256 * R;
    const int64_t n_tiles = (n + tile_samples - 1) / tile_samples;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * tile_samples + (int64_t)threadIdx.x * R;
        T x[DREG][R];
#pragma unroll
        for (int f = 0; f < DREG; ++f) {
            if (f < d) {
                load_row<T, R>(X_t + (size_t)f * n, i0, n, vec_ok != 0, x[f]);
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) x[f][r] = T(0);
            }
        }

        T best[R];
        uint32_t bi[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            best[r] = kmx_inf<T>();
            bi[r] = 0;
        }

        for (int c = 0; c < k; ++c) {
            const T* __restrict__ cp = cpack + (size_t)c * dpad;  // wave-uniform address
            T dot[R];
#pragma unroll
            for (int r = 0; r < R; ++r) dot[r] = T(0);
#pragma unroll
            for (int f4 = 0; f4 < DREG / 4; ++f4) {
                if (f4 * 4 < d) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const T cv = cp[f4 * 4 + j];
#pragma unroll
                        for (int r = 0; r < R; ++r) dot[r] = fma(x[f4 * 4 + j][r], cv, dot[r]);
                    }
                }
            }
            const T h = half_norms[c];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const T pd = h - dot[r];
                if (pd < best[r]) {
                    best[r] = pd;
                    bi[r] = (uint32_t)c;
                }
            }
        }

        // labels, changed-label count and accumulation
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t i = i0 + r;
            if (i < n) {
                labels[i] = bi[r];
                if (ACC != ACC_NONE) {
                    changed += (labels_prev[i] != bi[r]) ? 1u : 0u;
                    const T wr = sample_weight[i];
                    if (ACC == ACC_LDS) {
                        kmx_atomic_add(acc + (size_t)d * k + bi[r], (double)wr);
#pragma unroll
                        for (int f = 0; f < DREG; ++f) {
                            if (f < d) kmx_atomic_add(acc + (size_t)f * k + bi[r], (double)x[f][r] * (double)wr);
                        }
                    } else {
                        kmx_atomic_add(gacc + (size_t)d * k + bi[r], wr);
#pragma unroll
                        for (int f = 0; f < DREG; ++f) {
                            if (f < d) kmx_atomic_add(gacc + (size_t)f * k + bi[r], x[f][r] * wr);
                        }
                    }
                }
            }
        }
    }

    if (ACC != ACC_NONE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        if (ACC == ACC_LDS) {
            T* out = partial + (size_t)blockIdx.x * items;
            const double* all = reinterpret_cast<const double*>(smem_raw);
            for (int j = threadIdx.x; j < items; j += 256) {
                double tot = all[j];
                for (int c = 1; c < lds_copies; ++c) tot += all[(size_t)c * items + j];
                out[j] = (T)tot;
            }
        }
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
    }
}

// ------------------------------------------------------------------------------------------
// Streaming fused step for wide samples and few clusters: windows of KC centroids, features
// re-read per window (one window up to KC clusters).  A thread owns R consecutive samples and
// reads them with one 128-bit load per feature row.
// ------------------------------------------------------------------------------------------
template <typename T, int R, int KC, int ACC>
__global__ __launch_bounds__(256) void lloyd_fused_stream_kernel(
    const T* __restrict__ X_t, const T* __restrict__ sample_weight,
    const T* __restrict__ centroids_t, const T* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    T* __restrict__ partial, kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k,
    int n_copies, int vec_ok, int lds_copies) {
    if (status != nullptr && status->state != KMX_RUNNING) return;

    // LDS accumulators are fp64 for both types: ds_add_f64 is fast on this hardware, ds_add_f32
    // is not (about 195 cycles per wave instruction)
    extern __shared__ __align__(16) unsigned char smem_raw[];
    double* acc = reinterpret_cast<double*>(smem_raw);
    __shared__ unsigned int changed_block;
    const int items = (d + 1) * k;
    if (ACC == ACC_LDS) {
        for (int j = threadIdx.x; j < items * lds_copies; j += 256) acc[j] = 0.0;
        // few clusters mean many lanes of a wave on one address: lanes spread over copies
        acc += (size_t)(threadIdx.x & (lds_copies - 1)) * items;
    }
    if (threadIdx.x == 0) changed_block = 0;
    __syncthreads();

    T* gacc = (ACC == ACC_GLOBAL) ? partial + (size_t)(blockIdx.x % n_copies) * items : nullptr;
    unsigned int changed = 0;
    const int64_t tile_samples = 256 * R;
    const int64_t n_tiles = (n + tile_samples - 1) / tile_samples;

    for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int64_t i0 = tile * tile_samples + (int64_t)threadIdx.x * R;

        T best[R];
        uint32_t bi[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            best[r] = kmx_inf<T>();
            bi[r] = 0;
        }

        for (int c0 = 0; c0 < k; c0 += KC) {
            T dot[R][KC];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < KC; ++j) dot[r][j] = T(0);
#pragma unroll 4
            for (int f = 0; f < d; ++f) {
                T xv[R];
                load_row<T, R>(X_t + (size_t)f * n, i0, n, vec_ok != 0, xv);
                const T* __restrict__ crow = centroids_t + (size_t)f * k;  // wave-uniform
#pragma unroll
                for (int j = 0; j < KC; ++j) {
                    const int c = (c0 + j < k) ? c0 + j : k - 1;
                    const T cv = crow[c];
#pragma unroll
                    for (int r = 0; r < R; ++r) dot[r][j] = fma(xv[r], cv, dot[r][j]);
                }
            }
#pragma unroll
            for (int j = 0; j < KC; ++j) {
                if (c0 + j < k) {
                    const T h = half_norms[c0 + j];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const T pd = h - dot[r][j];
                        if (pd < best[r]) {
                            best[r] = pd;
                            bi[r] = (uint32_t)(c0 + j);
                        }
                    }
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; ++r)
            if (i0 + r < n) labels[i0 + r] = bi[r];

        if (ACC != ACC_NONE) {
            T wr[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const bool live = i0 + r < n;
                wr[r] = live ? sample_weight[i0 + r] : T(0);
                changed += (live && labels_prev[i0 + r] != bi[r]) ? 1u : 0u;
                if (live) {
                    if (ACC == ACC_LDS) kmx_atomic_add(acc + (size_t)d * k + bi[r], (double)wr[r]);
                    else kmx_atomic_add(gacc + (size_t)d * k + bi[r], wr[r]);
                }
            }
#pragma unroll 4
            for (int f = 0; f < d; ++f) {
                T xv[R];
                load_row<T, R>(X_t + (size_t)f * n, i0, n, vec_ok != 0, xv);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (i0 + r < n) {
                        if (ACC == ACC_LDS)
                            kmx_atomic_add(acc + (size_t)f * k + bi[r], (double)xv[r] * (double)wr[r]);
                        else
                            kmx_atomic_add(gacc + (size_t)f * k + bi[r], xv[r] * wr[r]);
                    }
                }
            }
        }
    }

    if (ACC != ACC_NONE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        if (ACC == ACC_LDS) {
            T* out = partial + (size_t)blockIdx.x * items;
            const double* all = reinterpret_cast<const double*>(smem_raw);
            for (int j = threadIdx.x; j < items; j += 256) {
                double tot = all[j];
                for (int c = 1; c < lds_copies; ++c) tot += all[(size_t)c * items + j];
                out[j] = (T)tot;
            }
        }
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
    }
}

// ------------------------------------------------------------------------------------------
// Reduction of the partial copies.  Block = 32 items x 8 copy lanes.  The last block to
// finish lists the empty clusters in ascending order and finds the heaviest cluster.
// ------------------------------------------------------------------------------------------
constexpr int RED_ITEMS = 16, RED_GROUPS = 16;  // 256 threads of the reduction kernel

template <typename T>
__global__ __launch_bounds__(256) void lloyd_reduce_kernel(
    T* __restrict__ partial, int n_partials, int clear_partials, T* __restrict__ sums_t,
    T* __restrict__ sizes, uint32_t* __restrict__ empty_clusters,
    kmx_lloyd_status* __restrict__ status, int d, int k,
    unsigned long long* __restrict__ gsum, const int* __restrict__ q_exp, int with_tail) {
    if (status->state != KMX_RUNNING) return;
    const int items = (d + 1) * k;
    if (gsum != nullptr) {
        // 64-bit fixed-point sums of the matrix-core step: converted and cleared by a grid-stride
        // loop of few blocks (every block ends with one atomic on the same ticket)
        for (int item = blockIdx.x * 256 + threadIdx.x; item < items; item += gridDim.x * 256) {
            const long long iv = (long long)gsum[item];
            gsum[item] = 0ull;
            const T v = (T)ldexp((double)iv, -q_exp[item / k]);
            if (item < d * k)
                sums_t[item] = v;
            else
                sizes[item - d * k] = v;
        }
    } else if (n_partials == 1) {
        // one copy of the sums (bucketed accumulation): moved and cleared by the same few blocks
        for (int item = blockIdx.x * 256 + threadIdx.x; item < items; item += gridDim.x * 256) {
            const T v = partial[item];
            if (clear_partials) partial[item] = T(0);
            if (item < d * k)
                sums_t[item] = v;
            else
                sizes[item - d * k] = v;
        }
    } else {
        // RED_ITEMS items per workgroup, RED_GROUPS thread groups over the partial slots
        // (fixed order: slot g + RED_GROUPS * i in thread group g, then the groups in order)
        const int it = threadIdx.x % RED_ITEMS;
        const int cl = threadIdx.x / RED_ITEMS;
        const int item = blockIdx.x * RED_ITEMS + it;
        __shared__ T red[RED_GROUPS][RED_ITEMS];
        T s = T(0);
        if (item < items) {
            for (int g = cl; g < n_partials; g += RED_GROUPS) {
                T* p = partial + (size_t)g * items + item;
                s += *p;
                if (clear_partials) *p = T(0);
            }
        }
        red[cl][it] = s;
        __syncthreads();
        if (cl == 0 && item < items) {
            T tot = red[0][it];
#pragma unroll
            for (int j = 1; j < RED_GROUPS; ++j) tot += red[j][it];
            if (item < d * k)
                sums_t[item] = tot;
            else
                sizes[item - d * k] = tot;
        }
    }

    // ---- last block: empty-cluster list + heaviest cluster (left to the one-workgroup
    // finalisation kernel when that one follows)
    if (!with_tail) return;
    __shared__ unsigned int is_last;
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int t = atomicAdd(&status->ticket, 1u);
        is_last = (t == gridDim.x - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();

    __shared__ int wave_counts[4];
    __shared__ T hv_val[4];
    __shared__ int hv_idx[4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int base = 0;
    T my_max = -kmx_inf<T>();
    int my_arg = 0x7fffffff;
    for (int c0 = 0; c0 < k; c0 += 256) {
        const int c = c0 + threadIdx.x;
        T sz = T(1);
        if (c < k) {
            sz = __builtin_nontemporal_load(sizes + c);
            if (sz > my_max) {
                my_max = sz;
                my_arg = c;
            }
        }
        const bool flag = (c < k) && (sz == T(0));
        const unsigned long long mask = __ballot(flag);
        const int prefix = __popcll(mask & ((1ull << lane) - 1ull));
        if (lane == 0) wave_counts[wave] = __popcll(mask);
        __syncthreads();
        int offset = base;
        for (int w2 = 0; w2 < wave; ++w2) offset += wave_counts[w2];
        if (flag) empty_clusters[offset + prefix] = (uint32_t)c;
        base += wave_counts[0] + wave_counts[1] + wave_counts[2] + wave_counts[3];
        __syncthreads();
    }
    // heaviest cluster, lowest index on ties
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const T ov = __shfl_xor(my_max, off, 64);
        const int oi = __shfl_xor(my_arg, off, 64);
        if (ov > my_max || (ov == my_max && oi < my_arg)) {
            my_max = ov;
            my_arg = oi;
        }
    }
    if (lane == 0) {
        hv_val[wave] = my_max;
        hv_idx[wave] = my_arg;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        T bv = hv_val[0];
        int bidx = hv_idx[0];
        for (int w2 = 1; w2 < 4; ++w2) {
            if (hv_val[w2] > bv || (hv_val[w2] == bv && hv_idx[w2] < bidx)) {
                bv = hv_val[w2];
                bidx = hv_idx[w2];
            }
        }
        status->reserved[0] = bidx;
        status->n_empty = base;
        status->ticket = 0;
        if (base > 0) status->state = KMX_NEED_RELOCATION;
    }
}

// ------------------------------------------------------------------------------------------
// Finalisation: LANES threads per cluster (256 / LANES clusters per workgroup), lane g on the
// features g, g + LANES, ... (division, packed copy, half squared norm, squared shift); the lanes
// meet in LDS in lane order.  8 lanes, or 64 for a few clusters of wide samples, where a
// workgroup or two of eight-lane clusters would each walk a hundred features, a trip to memory
// per value.  The last block sums the per-block shifts in block order and runs the convergence
// test.
// ------------------------------------------------------------------------------------------
constexpr int fin_lanes(int d, int k) { return (d >= 256 && k <= 128) ? 64 : 8; }
constexpr int fin_grid(int d, int k) { return (k + 256 / fin_lanes(d, k) - 1) / (256 / fin_lanes(d, k)); }

template <typename T, int LANES>
__global__ __launch_bounds__(256) void lloyd_finalize_kernel(
    const T* __restrict__ old_centroids_t, T* __restrict__ new_centroids_t,
    const T* __restrict__ sizes, T* __restrict__ cpack, T* __restrict__ half_norms,
    double* __restrict__ shift_partial, kmx_lloyd_status* __restrict__ status, int d, int k,
    int dpad, int force) {
    const int state = status->state;
    if (force ? (state != KMX_NEED_RELOCATION && state != KMX_RUNNING) : (state != KMX_RUNNING))
        return;
    constexpr int CPW = 256 / LANES;  // clusters per workgroup
    const int cl = threadIdx.x & (CPW - 1), grp = threadIdx.x / CPW;
    const int c = blockIdx.x * CPW + cl;
    __shared__ T sq_s[LANES][CPW], sh_s[LANES][CPW];
    T sq = T(0), sh = T(0);
    const T sz = c < k ? sizes[c] : T(0);
    if (sz != T(0)) {
#pragma unroll 4
        for (int f = grp; f < d; f += LANES) {
            const T nv = new_centroids_t[(size_t)f * k + c] / sz;
            const T df = old_centroids_t[(size_t)f * k + c] - nv;
            sh += df * df;
            sq += nv * nv;
            cpack[(size_t)c * dpad + f] = nv;
            new_centroids_t[(size_t)f * k + c] = nv;
        }
        for (int f = d + grp; f < dpad; f += LANES) cpack[(size_t)c * dpad + f] = T(0);
    }
    sq_s[grp][cl] = sq;
    sh_s[grp][cl] = sh;
    __syncthreads();
    double shift = 0.0;
    if (grp == 0 && sz != T(0)) {
        T sq_t = sq_s[0][cl], sh_t = sh_s[0][cl];
#pragma unroll
        for (int g2 = 1; g2 < LANES; ++g2) {
            sq_t += sq_s[g2][cl];
            sh_t += sh_s[g2][cl];
        }
        half_norms[c] = sq_t / T(2);
        shift = (double)sh_t;
    }
    __shared__ double scratch[4];
    const double block_shift = kmx_block_sum<double>(shift, scratch);
    __shared__ unsigned int is_last;
    if (threadIdx.x == 0) {
        shift_partial[blockIdx.x] = block_shift;
        __threadfence();
        const unsigned int t = atomicAdd(&status->ticket, 1u);
        is_last = (t == gridDim.x - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();

    // Clusters that are still empty (more clusters than distinct samples, so nothing could
    // be relocated) are parked on the finished centroid of the heaviest cluster.
    double parked_shift = 0.0;
    if (status->n_empty > 0) {
        const int heaviest = (int)status->reserved[0];
        for (int c2 = threadIdx.x; c2 < k; c2 += 256) {
            if (sizes[c2] == T(0)) {
                T sq = T(0), sh = T(0);
                for (int f = 0; f < d; ++f) {
                    const T nv = __builtin_nontemporal_load(cpack + (size_t)heaviest * dpad + f);
                    const T df = old_centroids_t[(size_t)f * k + c2] - nv;
                    sh += df * df;
                    sq += nv * nv;
                    cpack[(size_t)c2 * dpad + f] = nv;
                    new_centroids_t[(size_t)f * k + c2] = nv;
                }
                for (int f = d; f < dpad; ++f) cpack[(size_t)c2 * dpad + f] = T(0);
                half_norms[c2] = sq / T(2);
                parked_shift += (double)sh;
            }
        }
    }
    parked_shift = kmx_block_sum<double>(parked_shift, scratch);
    if (threadIdx.x == 0) {
        double total = parked_shift;
        for (unsigned int b = 0; b < gridDim.x; ++b)
            total += __builtin_nontemporal_load(shift_partial + b);
        const int n_iter = status->n_iter + 1;
        const unsigned int changed = status->n_changed;
        status->n_iter = n_iter;
        status->shift_sum = total;
        status->n_changed = 0;
        status->ticket = 0;
        int next = KMX_RUNNING;
        if (n_iter > 1 && changed == 0)
            next = KMX_CONVERGED_STRICT;
        else if (!(total > status->tol))
            next = KMX_CONVERGED_TOL;
        else if (n_iter >= status->max_iter)
            next = KMX_MAX_ITER;
        status->state = next;
        status->reserved[1] = (int64_t)changed;
    }
}

// Packed (k, dpad) copy of the centroids + half squared norms; optional status reset.
// LANES feature lanes per cluster (256 / LANES clusters per workgroup): lane g of a cluster takes
// the features g, g + LANES, ...; 8 lanes, or 64 for wide samples, where eight lanes would each
// walk a hundred features, a trip to memory per value.
template <typename T, int LANES>
__global__ __launch_bounds__(256) void lloyd_pack_kernel(const T* __restrict__ centroids_t,
                                                         T* __restrict__ cpack,
                                                         T* __restrict__ half_norms,
                                                         kmx_lloyd_status* __restrict__ status,
                                                         int d, int k, int dpad, int max_iter,
                                                         double tol) {
    const int g = threadIdx.x & (LANES - 1);
    const int c = blockIdx.x * (256 / LANES) + (int)(threadIdx.x / LANES);
    T sq = T(0);
    if (c < k) {
        if constexpr (LANES == 8) {
            for (int f = g; f < dpad; f += 8) {
                const T v = f < d ? centroids_t[(size_t)f * k + c] : T(0);
                sq += v * v;
                cpack[(size_t)c * dpad + f] = v;
            }
        } else {
            // (eight loads in flight, then their stores)
            for (int f0 = g; f0 < dpad; f0 += 8 * LANES) {
                T v[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int f = f0 + u * LANES;
                    v[u] = f < d ? centroids_t[(size_t)f * k + c] : T(0);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int f = f0 + u * LANES;
                    sq += v[u] * v[u];
                    if (f < dpad) cpack[(size_t)c * dpad + f] = v[u];
                }
            }
        }
    }
#pragma unroll
    for (int off = 1; off < LANES; off <<= 1) sq += __shfl_xor(sq, off, 64);
    if (c < k && g == 0) half_norms[c] = sq / T(2);
    if (status != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
        status->n_iter = 0;
        status->state = max_iter > 0 ? KMX_RUNNING : KMX_MAX_ITER;
        status->n_empty = 0;
        status->n_changed = 0;
        status->shift_sum = __builtin_huge_val();
        status->tol = tol;
        status->max_iter = max_iter;
        status->ticket = 0;
        status->max_sq_dist = 0.0;
        status->reserved[0] = 0;
        status->reserved[1] = 0;
    }
}

template <typename T>
static void launch_pack(const void* centroids_t, void* cpack, void* half_norms, kmx_lloyd_status* status, int d, int k,
                        int dpad, int max_iter, double tol, hipStream_t stream) {
    if (d >= 256)
        hipLaunchKernelGGL((lloyd_pack_kernel<T, 64>), dim3((unsigned)kmx_cdiv(k, 4)), dim3(256), 0, stream,
                           (const T*)centroids_t, (T*)cpack, (T*)half_norms, status, d, k, dpad, max_iter, tol);
    else
        hipLaunchKernelGGL((lloyd_pack_kernel<T, 8>), dim3((unsigned)kmx_cdiv(k, 32)), dim3(256), 0, stream,
                           (const T*)centroids_t, (T*)cpack, (T*)half_norms, status, d, k, dpad, max_iter, tol);
}

__global__ void fill_zero_bytes_kernel(uint32_t* __restrict__ p, size_t n_words) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride)
        p[i] = 0u;
}

// ------------------------------------------------------------------------------------------
// Host-side launchers
// ------------------------------------------------------------------------------------------

// Samples per thread of the streaming kernel: one 128-bit load per feature row, or single
// samples while that would leave compute units without a workgroup.
static int lloyd_stream_samples_per_thread(int64_t n, int dtype) {
    const int rv = dtype == KMX_F32 ? 4 : 2;
    return n >= (int64_t)256 * rv * 2 * kmx_num_cus() ? rv : 1;
}

// Workgroups of a vector-ALU fused step (also the number of partial slots it fills).
int lloyd_fused_grid(const LloydLayout& L, int64_t n, int d, int dtype) {
    if (L.variant == KMX_VARIANT_MFMA_F64) return kmx_mfma_f64_grid(n, d, L.wgs_per_cu, L.cols, L.partial_slots());
    if (L.variant == KMX_VARIANT_FEWK) return kmx_fewk_grid(n, d, L.k_for_gsum, L.wgs_per_cu);
    const int r = (L.variant == KMX_VARIANT_REGISTER) ? lloyd_reg_samples_per_thread(d, dtype)
                                                      : lloyd_stream_samples_per_thread(n, dtype);
    const int64_t tiles = kmx_cdiv(n, 256 * (int64_t)r);
    const int cap = L.grid_cap(kmx_num_cus());
    int grid = (int)(tiles < cap ? tiles : cap);
    return grid < 1 ? 1 : grid;
}

// Copies of the LDS accumulators of the vector-ALU kernels (a power of two, at most 8, within
// KMX_LDS_ACC_LIMIT): with k clusters a wave's atomics of one feature fall on k addresses.
static int lds_acc_copies(int d, int k) {
    const size_t one = (size_t)(d + 1) * k * sizeof(double);
    int copies = 1;
    while (copies < 8 && copies * 2 * (size_t)k <= 64 && one * copies * 2 <= KMX_LDS_ACC_LIMIT) copies *= 2;
    return copies;
}

template <typename T, int DREG, int R, int ACC>
void launch_reg(const LloydLayout& L, const void* X_t, const void* w, const T* cpack,
                const T* half_norms, const uint32_t* labels_prev, uint32_t* labels, T* partial,
                kmx_lloyd_status* status, int64_t n, int d, int k, int grid, hipStream_t stream) {
    const int copies = lds_acc_copies(d, k);
    const size_t lds = (ACC == ACC_LDS) ? (size_t)(d + 1) * k * sizeof(double) * copies : 0;
    const int vec_ok = (n % R == 0) && (((uintptr_t)X_t) % (R * sizeof(T)) == 0);
    hipLaunchKernelGGL((lloyd_fused_reg_kernel<T, DREG, R, ACC>), dim3(grid), dim3(256), lds, stream,
                       (const T*)X_t, (const T*)w, cpack, half_norms, labels_prev, labels, partial,
                       status, n, d, k, L.dpad, L.n_partials, vec_ok, copies);
}

// Returns the status of the entry point it hands over to (a refusal there would leave `labels`
// unwritten, and the sums kernels that follow index LDS and memory with them).
template <typename T, int ACC>
int32_t launch_fused(const LloydLayout& L, const void* X_t, const void* w, const void* centroids_t,
                  const T* cpack, const T* half_norms, const uint32_t* labels_prev,
                  uint32_t* labels, T* partial, kmx_lloyd_status* status, int64_t n, int d, int k,
                  hipStream_t stream, const unsigned int* screen_absmax = nullptr, char* screen_area = nullptr,
                  const void* X_rowmajor = nullptr) {
    const int grid = lloyd_fused_grid(L, n, d, sizeof(T) == 8 ? KMX_F64 : KMX_F32);
    if (L.variant == KMX_VARIANT_GEMM) {
        if (sizeof(T) == 4 && L.screen_labels)
            return kmx_lloyd_labels_mfma_screen(X_t, centroids_t, labels, status, n, d, k, L.wgs_per_cu, stream);
        else if (sizeof(T) == 4 && L.gemm_screen && screen_area != nullptr)
            return kmx_lloyd_gemm_screen_labels(X_t, centroids_t, half_norms, screen_absmax, screen_area, labels,
                                                status, n, d, k, stream);
        else
            return kmx_lloyd_gemm_labels(X_t, centroids_t, half_norms, labels, status, n, d, k,
                                         sizeof(T) == 8 ? KMX_F64 : KMX_F32, stream);
    } else if (L.variant == KMX_VARIANT_MFMA_F64) {
        return kmx_lloyd_step_mfma_f64(X_t, w, centroids_t, half_norms, labels_prev, labels, partial,
                                       status, n, d, k, ACC != ACC_NONE, L.wgs_per_cu, L.cols, L.partial_slots(),
                                       stream);
    } else if (L.variant == KMX_VARIANT_REGISTER) {
#define KMX_REG_CASE(DR, RR)                                                                    \
    launch_reg<T, DR, RR, ACC>(L, X_t, w, cpack, half_norms, labels_prev, labels, partial, status, \
                               n, d, k, grid, stream)
        if constexpr (sizeof(T) == 4) {
            if (d <= 8)
                KMX_REG_CASE(8, 4);
            else if (d <= 16)
                KMX_REG_CASE(16, 4);
            else if (d <= 32)
                KMX_REG_CASE(32, 2);
            else
                KMX_REG_CASE(64, 1);
        } else {
            if (d <= 8)
                KMX_REG_CASE(8, 2);
            else if (d <= 16)
                KMX_REG_CASE(16, 2);
            else if (d <= 32)
                KMX_REG_CASE(32, 1);
            else
                KMX_REG_CASE(64, 1);
        }
#undef KMX_REG_CASE
    } else {
        constexpr int RV = 16 / (int)sizeof(T), KC = 16;
        const int copies = lds_acc_copies(d, k);
        const size_t lds = (ACC == ACC_LDS) ? (size_t)(d + 1) * k * sizeof(double) * copies : 0;
        if (lloyd_stream_samples_per_thread(n, sizeof(T) == 8 ? KMX_F64 : KMX_F32) == 1) {
            hipLaunchKernelGGL((lloyd_fused_stream_kernel<T, 1, KC, ACC>), dim3(grid), dim3(256), lds,
                               stream, (const T*)X_t, (const T*)w, (const T*)centroids_t, half_norms,
                               labels_prev, labels, partial, status, n, d, k, L.n_partials, 0, copies);
        } else {
            const int vec_ok = (n % RV == 0) && (((uintptr_t)X_t) % 16 == 0);
            hipLaunchKernelGGL((lloyd_fused_stream_kernel<T, RV, KC, ACC>), dim3(grid), dim3(256), lds,
                               stream, (const T*)X_t, (const T*)w, (const T*)centroids_t, half_norms,
                               labels_prev, labels, partial, status, n, d, k, L.n_partials, vec_ok, copies);
        }
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

template <typename T>
int32_t lloyd_iter_impl(const LloydLayout& L, const void* X_t, const void* X_rowmajor, const void* w,
                        const void* centroids_t, void* new_centroids_t,
                        const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                        uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                        hipStream_t stream, hipEvent_t* events = nullptr) {
    auto* status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    T* cpack = reinterpret_cast<T*>(ws + L.off_cpack);
    T* half_norms = reinterpret_cast<T*>(ws + L.off_half);
    T* partial = reinterpret_cast<T*>(ws + L.off_partial);
    double* shift_partial = reinterpret_cast<double*>(ws + L.off_shift);

    if (events) (void)hipEventRecord(events[0], stream);
    int n_partials_used = L.n_partials;
    unsigned long long* gsum = nullptr;
    const int* q_exp = nullptr;
    if (L.variant == KMX_VARIANT_MFMA_WIDE) {
        if constexpr (sizeof(T) == 4) {
            const int32_t rc = kmx_lloyd_step_mfma_wide_f32(L, X_t, X_rowmajor, w, centroids_t,
                                                            labels_prev, labels, ws, n, d, k, stream);
            if (rc != KMX_OK) return rc;
        }
        gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
        q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
    } else if (L.acc_mode == KMX_ACC_BUCKET) {
        const int32_t rc_labels =
            launch_fused<T, ACC_NONE>(L, X_t, w, centroids_t, cpack, half_norms, labels_prev, labels,
                                      partial, status, n, d, k, stream,
                                      reinterpret_cast<const unsigned int*>(ws + L.off_scales), ws + L.off_wscreen);
        if (rc_labels != KMX_OK) return rc_labels;
        if (sizeof(T) == 4 && L.direct_sums) {
            gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
            q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
            const int32_t rc = kmx_lloyd_direct_sums(X_t, w, labels_prev, labels, q_exp, gsum, status, n, d, k,
                                                     stream);
            if (rc != KMX_OK) return rc;
        } else {
            const int32_t rc = kmx_lloyd_bucket_sums(X_t, X_rowmajor, w, labels_prev, labels, partial, status,
                                                     ws + L.off_bucket, n, d, k,
                                                     sizeof(T) == 8 ? KMX_F64 : KMX_F32, stream);
            if (rc != KMX_OK) return rc;
        }
    } else if (L.acc_mode == ACC_LDS) {
        const int32_t rc_step =
            launch_fused<T, ACC_LDS>(L, X_t, w, centroids_t, cpack, half_norms, labels_prev, labels,
                                     partial, status, n, d, k, stream, nullptr, nullptr, X_rowmajor);
        if (rc_step != KMX_OK) return rc_step;
        n_partials_used = lloyd_fused_grid(L, n, d, sizeof(T) == 8 ? KMX_F64 : KMX_F32);
    } else {
        const int32_t rc_step =
            launch_fused<T, ACC_GLOBAL>(L, X_t, w, centroids_t, cpack, half_norms, labels_prev, labels,
                                        partial, status, n, d, k, stream);
        if (rc_step != KMX_OK) return rc_step;
    }
    KMX_LAUNCH_CHECK();
    if (events) (void)hipEventRecord(events[1], stream);
    const int items = (d + 1) * k;
    if constexpr (sizeof(T) == 4) {
        if (L.direct_sums && items <= 6 * 1024) {
            // few fixed-point sums: converted, cleared and finished by one workgroup (measured:
            // 9 us for 1 900 sums, 27 us for 10 500; the conversion pass and the general
            // finalisation below take 18 us for 16 600)
            if (events) (void)hipEventRecord(events[2], stream);
            LloydTail<float> tail;
            tail.sums_t = (float*)new_centroids_t;
            tail.sizes = (float*)sizes;
            tail.empty_clusters = empty_clusters;
            tail.old_centroids_t = (const float*)centroids_t;
            tail.cpack = cpack;
            tail.half_norms = half_norms;
            tail.status = status;
            tail.d = d;
            tail.k = k;
            tail.dpad = L.dpad;
            hipLaunchKernelGGL((lloyd_small_finalize_kernel<float, true>), dim3(1), dim3(256),
                               (size_t)items * sizeof(float), stream, gsum, q_exp, tail);
            KMX_LAUNCH_CHECK();
            if (events) (void)hipEventRecord(events[3], stream);
            return KMX_OK;
        }
    }
    const int64_t reduce_grid = (gsum != nullptr || n_partials_used == 1)
                                    ? (kmx_cdiv(items, 256) < 128 ? kmx_cdiv(items, 256) : 128)
                                    : kmx_cdiv(items, RED_ITEMS);
    // sums that fit in LDS are finished by one workgroup (no device-wide fences or tickets)
    const bool small_tail = gsum == nullptr && items <= 6 * 1024;
    hipLaunchKernelGGL((lloyd_reduce_kernel<T>), dim3((unsigned)reduce_grid), dim3(256), 0,
                       stream, partial, n_partials_used,
                       ((L.acc_mode == ACC_GLOBAL || L.acc_mode == KMX_ACC_BUCKET) && gsum == nullptr) ? 1 : 0,
                       (T*)new_centroids_t, (T*)sizes, empty_clusters, status, d, k, gsum, q_exp,
                       small_tail ? 0 : 1);
    KMX_LAUNCH_CHECK();
    if (events) (void)hipEventRecord(events[2], stream);
    if (small_tail) {
        LloydTail<T> tail;
        tail.sums_t = (T*)new_centroids_t;
        tail.sizes = (T*)sizes;
        tail.empty_clusters = empty_clusters;
        tail.old_centroids_t = (const T*)centroids_t;
        tail.cpack = cpack;
        tail.half_norms = half_norms;
        tail.status = status;
        tail.d = d;
        tail.k = k;
        tail.dpad = L.dpad;
        hipLaunchKernelGGL((lloyd_small_finalize_kernel<T, false>), dim3(1), dim3(256),
                           (size_t)items * sizeof(T), stream, nullptr, nullptr, tail);
    } else {
        if (fin_lanes(d, k) == 64)
            hipLaunchKernelGGL((lloyd_finalize_kernel<T, 64>), dim3((unsigned)fin_grid(d, k)), dim3(256), 0,
                               stream, (const T*)centroids_t, (T*)new_centroids_t, (const T*)sizes, cpack,
                               half_norms, shift_partial, status, d, k, L.dpad, 0);
        else
            hipLaunchKernelGGL((lloyd_finalize_kernel<T, 8>), dim3((unsigned)fin_grid(d, k)), dim3(256), 0,
                               stream, (const T*)centroids_t, (T*)new_centroids_t, (const T*)sizes, cpack,
                               half_norms, shift_partial, status, d, k, L.dpad, 0);
    }
    KMX_LAUNCH_CHECK();
    if (events) (void)hipEventRecord(events[3], stream);
    return KMX_OK;
}

}  // namespace

// ------------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------------

int32_t kmx_num_cus() {
    static int32_t cached = 0;
    if (cached > 0) return cached;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
        return 256;
    cached = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    return cached;
}

extern "C" {

int32_t kmx_abi_version(void) { return KMX_ABI_VERSION; }

const char* kmx_error_string(int32_t code) {
    switch (code) {
        case KMX_OK: return "ok";
        case KMX_ERR_NULL_POINTER: return "null pointer argument";
        case KMX_ERR_BAD_SHAPE: return "invalid or inconsistent shape";
        case KMX_ERR_BAD_DTYPE: return "dtype must be KMX_F32 (0) or KMX_F64 (1)";
        case KMX_ERR_WORKSPACE: return "workspace too small";
        case KMX_ERR_BAD_ARGUMENT: return "invalid argument";
        case KMX_ERR_UNSUPPORTED: return "shape not supported by this kernel";
        case KMX_ERR_BAD_PLAN: return "kmx_lloyd_plan not made by kmx_lloyd_plan_init of this library, or edited";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}

// ---- plan: shape + flags + what follows from them; validated by every call that takes one

static uint64_t plan_check_value(const kmx_lloyd_plan& p) {
    // FNV-1a over the fields in declaration order (not over padding)
    uint64_t h = 1469598103934665603ull;
    auto mix = [&h](uint64_t v) {
        for (int i = 0; i < 8; ++i) {
            h ^= (v >> (8 * i)) & 0xffu;
            h *= 1099511628211ull;
        }
    };
    mix(p.magic);
    mix((uint64_t)(uint32_t)p.abi_version);
    mix((uint64_t)p.n);
    mix((uint64_t)(uint32_t)p.d);
    mix((uint64_t)(uint32_t)p.k);
    mix((uint64_t)(uint32_t)p.dtype);
    mix(p.flags);
    mix((uint64_t)(uint32_t)p.variant);
    mix((uint64_t)(uint32_t)p.reserved);
    mix(p.workspace_bytes);
    return h;
}
constexpr uint32_t KMX_PLAN_MAGIC = 0x50584d4bu;  // "KMXP"

static int32_t plan_validate(const kmx_lloyd_plan* p) {
    if (p == nullptr) return KMX_ERR_NULL_POINTER;
    if (p->magic != KMX_PLAN_MAGIC || p->abi_version != KMX_ABI_VERSION || p->check != plan_check_value(*p))
        return KMX_ERR_BAD_PLAN;
    return KMX_OK;
}
#define KMX_REQUIRE_PLAN(p)                     \
    do {                                        \
        const int32_t rc_ = plan_validate(p);   \
        if (rc_ != KMX_OK) return rc_;          \
    } while (0)

static int32_t layout_variant_code(const LloydLayout& L) {
    return L.screen ? 61 : L.screen64 ? 71 : L.variant * 10 + L.acc_mode;
}

int32_t kmx_lloyd_plan_init(kmx_lloyd_plan* plan, int64_t n, int32_t d, int32_t k, int32_t dtype,
                            uint32_t flags) {
    KMX_REQUIRE_PTR(plan);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (!kmx_flags_valid(flags)) return KMX_ERR_BAD_ARGUMENT;
    const LloydLayout L = lloyd_layout(n, d, k, dtype, flags);
    plan->magic = KMX_PLAN_MAGIC;
    plan->abi_version = KMX_ABI_VERSION;
    plan->n = n;
    plan->d = d;
    plan->k = k;
    plan->dtype = dtype;
    plan->flags = flags;
    plan->variant = layout_variant_code(L);
    plan->reserved = 0;
    plan->workspace_bytes = L.total;
    plan->check = plan_check_value(*plan);
    return KMX_OK;
}

size_t kmx_lloyd_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags) {
    kmx_lloyd_plan plan;
    return kmx_lloyd_plan_init(&plan, n, d, k, dtype, flags) == KMX_OK ? (size_t)plan.workspace_bytes : 0;
}

int32_t kmx_lloyd_kernel_variant(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags) {
    kmx_lloyd_plan plan;
    const int32_t rc = kmx_lloyd_plan_init(&plan, n, d, k, dtype, flags);
    return rc == KMX_OK ? plan.variant : rc;
}

int32_t kmx_lloyd_plan_reads_rowmajor(const kmx_lloyd_plan* plan) {
    KMX_REQUIRE_PLAN(plan);
    const LloydLayout L = lloyd_layout(plan->n, plan->d, plan->k, plan->dtype, plan->flags);
    if (L.variant == KMX_VARIANT_MFMA_WIDE || L.variant == KMX_VARIANT_FEWK) return 1;
    return (L.acc_mode == KMX_ACC_BUCKET && !L.direct_sums) ? 1 : 0;
}

int32_t kmx_lloyd_init(const kmx_lloyd_plan* plan, void* workspace, size_t workspace_bytes,
                       const void* X_t, const void* sample_weight, const void* centroids_t,
                       int32_t max_iter, double tol, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PLAN(plan);
    KMX_REQUIRE_PTR(workspace);
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(sample_weight);
    KMX_REQUIRE_PTR(centroids_t);
    if (max_iter < 0) return KMX_ERR_BAD_SHAPE;
    const int64_t n = plan->n;
    const int32_t d = plan->d, k = plan->k, dtype = plan->dtype;
    const LloydLayout L = lloyd_layout(n, d, k, dtype, plan->flags);
    if (workspace_bytes < L.total) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    char* ws = (char*)workspace;
    auto* status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    if (dtype == KMX_F32)
        launch_pack<float>(centroids_t, ws + L.off_cpack, ws + L.off_half, status, d, k, L.dpad, max_iter, tol, stream);
    else
        launch_pack<double>(centroids_t, ws + L.off_cpack, ws + L.off_half, status, d, k, L.dpad, max_iter, tol, stream);
    KMX_LAUNCH_CHECK();
    if (L.variant == KMX_VARIANT_MFMA || L.variant == KMX_VARIANT_MFMA_WIDE || L.gemm_screen || L.direct_sums ||
        L.screen64 || L.variant == KMX_VARIANT_FEWK) {
        // (for the screened tiled product: max|x| per feature, from which its scale is taken)
        const int32_t rc = kmx_lloyd_mfma_prepare(L, X_t, sample_weight, ws, n, d, dtype, stream);
        if (rc != KMX_OK) return rc;
    }
    if (L.variant == KMX_VARIANT_MFMA_WIDE || L.screen || L.screen64) {
        // cluster counts of the wide path / the counter of uncertain samples of the screened one
        hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(4), dim3(256), 0, stream,
                           (uint32_t*)(ws + L.off_bucket),
                           (L.screen || L.screen64) ? (size_t)64 : (size_t)k);
        KMX_LAUNCH_CHECK();
    }
    if (L.variant == KMX_VARIANT_MFMA_WIDE) {
        hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(1), dim3(64), 0, stream,
                           (uint32_t*)(ws + L.off_wscreen), (size_t)64);
        KMX_LAUNCH_CHECK();
    }
    if (L.acc_mode == KMX_ACC_BUCKET) {
        hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(4), dim3(256), 0, stream,
                           (uint32_t*)(ws + L.off_bucket), (size_t)k);
        KMX_LAUNCH_CHECK();
    }
    if ((L.acc_mode == ACC_GLOBAL || L.acc_mode == KMX_ACC_BUCKET) && L.partial_bytes > 0) {
        const size_t words = L.partial_bytes / 4;
        hipLaunchKernelGGL(fill_zero_bytes_kernel, dim3(1024), dim3(256), 0, stream,
                           (uint32_t*)(ws + L.off_partial), words);
        KMX_LAUNCH_CHECK();
    }
    return KMX_OK;
}

static int32_t lloyd_iter_dispatch(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                                   const void* sample_weight, const void* centroids_t,
                                   void* new_centroids_t,
                                   const uint32_t* labels_prev, uint32_t* labels,
                                   void* cluster_sizes, uint32_t* empty_clusters, void* workspace,
                                   size_t workspace_bytes, void* stream_, hipEvent_t* events) {
    KMX_REQUIRE_PLAN(plan);
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(sample_weight);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(new_centroids_t);
    KMX_REQUIRE_PTR(labels_prev);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(cluster_sizes);
    KMX_REQUIRE_PTR(empty_clusters);
    KMX_REQUIRE_PTR(workspace);
    const int64_t n = plan->n;
    const int32_t d = plan->d, k = plan->k, dtype = plan->dtype;
    const LloydLayout L = lloyd_layout(n, d, k, dtype, plan->flags);
    if (workspace_bytes < L.total) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32) {
        if (L.variant == KMX_VARIANT_MFMA)
            return kmx_lloyd_iter_mfma_f32(L, X_t, sample_weight, centroids_t, new_centroids_t,
                                           labels_prev, labels, cluster_sizes, empty_clusters,
                                           (char*)workspace, n, d, k, stream, events);
        if (L.variant == KMX_VARIANT_FEWK)
            return kmx_lloyd_iter_fewk(L, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t, labels_prev,
                                       labels, cluster_sizes, empty_clusters, (char*)workspace, n, d, k, stream,
                                       events);
        return lloyd_iter_impl<float>(L, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t,
                                      labels_prev, labels, cluster_sizes, empty_clusters,
                                      (char*)workspace, n, d, k, stream, events);
    }
    if (L.screen64)
        return kmx_lloyd_iter_mfma_screen_f64(L, X_t, sample_weight, centroids_t, new_centroids_t, labels_prev,
                                              labels, cluster_sizes, empty_clusters, (char*)workspace, n, d, k,
                                              stream, events);
    return lloyd_iter_impl<double>(L, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t, labels_prev,
                                   labels, cluster_sizes, empty_clusters, (char*)workspace, n, d, k,
                                   stream, events);
}

int32_t kmx_lloyd_iter(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                       const void* sample_weight, const void* centroids_t, void* new_centroids_t,
                       const uint32_t* labels_prev, uint32_t* labels, void* cluster_sizes,
                       uint32_t* empty_clusters, void* workspace, size_t workspace_bytes,
                       void* stream_) {
    KMX_ENTRY();
    return lloyd_iter_dispatch(plan, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t, labels_prev,
                               labels, cluster_sizes, empty_clusters, workspace, workspace_bytes, stream_,
                               nullptr);
}

int32_t kmx_lloyd_iter_timed(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                             const void* sample_weight, const void* centroids_t,
                             void* new_centroids_t, const uint32_t* labels_prev, uint32_t* labels,
                             void* cluster_sizes, uint32_t* empty_clusters, void* workspace,
                             size_t workspace_bytes, void* stream_, float* kernel_ms_host) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(kernel_ms_host);
    KMX_REQUIRE_PLAN(plan);
    hipEvent_t ev[4];
    for (int i = 0; i < 4; ++i) {
        const hipError_t e = hipEventCreate(&ev[i]);
        if (e != hipSuccess) return (int32_t)e;
    }
    int32_t rc = lloyd_iter_dispatch(plan, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t,
                                     labels_prev, labels, cluster_sizes, empty_clusters, workspace,
                                     workspace_bytes, stream_, ev);
    if (rc == KMX_OK) {
        hipError_t e = hipEventSynchronize(ev[3]);
        for (int i = 0; i < 3 && e == hipSuccess; ++i)
            e = hipEventElapsedTime(&kernel_ms_host[i], ev[i], ev[i + 1]);
        if (e != hipSuccess) rc = (int32_t)e;
    }
    for (int i = 0; i < 4; ++i) (void)hipEventDestroy(ev[i]);
    return rc;
}

// Events of the launches that kmx_lloyd_iter_traced has enqueued and kmx_lloyd_trace_collect has
// not yet read: four per launch.
static std::mutex trace_mutex;
static std::vector<hipEvent_t> trace_events;
constexpr size_t KMX_TRACE_MAX_LAUNCHES = 1024;

int32_t kmx_lloyd_iter_traced(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                              const void* sample_weight, const void* centroids_t,
                              void* new_centroids_t, const uint32_t* labels_prev, uint32_t* labels,
                              void* cluster_sizes, uint32_t* empty_clusters, void* workspace,
                              size_t workspace_bytes, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PLAN(plan);
    std::lock_guard<std::mutex> guard(trace_mutex);
    if (trace_events.size() >= 4 * KMX_TRACE_MAX_LAUNCHES) return KMX_ERR_UNSUPPORTED;
    hipEvent_t ev[4];
    for (int i = 0; i < 4; ++i) {
        const hipError_t e = hipEventCreate(&ev[i]);
        if (e != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipEventDestroy(ev[j]);
            return (int32_t)e;
        }
    }
    const int32_t rc = lloyd_iter_dispatch(plan, X_t, X_rowmajor, sample_weight, centroids_t, new_centroids_t,
                                           labels_prev, labels, cluster_sizes, empty_clusters, workspace,
                                           workspace_bytes, stream_, ev);
    if (rc != KMX_OK) {
        for (int i = 0; i < 4; ++i) (void)hipEventDestroy(ev[i]);
        return rc;
    }
    trace_events.insert(trace_events.end(), ev, ev + 4);
    return KMX_OK;
}

int32_t kmx_lloyd_trace_collect(float* kernel_ms_mean, float* kernel_ms_min, int32_t* n_launches) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(kernel_ms_mean);
    KMX_REQUIRE_PTR(n_launches);
    std::lock_guard<std::mutex> guard(trace_mutex);
    const size_t launches = trace_events.size() / 4;
    *n_launches = (int32_t)launches;
    double sum[3] = {0.0, 0.0, 0.0};
    float low[3] = {0.0f, 0.0f, 0.0f};
    int32_t rc = KMX_OK;
    for (size_t l = 0; l < launches && rc == KMX_OK; ++l) {
        hipError_t e = hipEventSynchronize(trace_events[4 * l + 3]);
        for (int i = 0; i < 3 && e == hipSuccess; ++i) {
            float ms = 0.0f;
            e = hipEventElapsedTime(&ms, trace_events[4 * l + i], trace_events[4 * l + i + 1]);
            sum[i] += ms;
            if (l == 0 || ms < low[i]) low[i] = ms;
        }
        if (e != hipSuccess) rc = (int32_t)e;
    }
    for (hipEvent_t ev : trace_events) (void)hipEventDestroy(ev);
    trace_events.clear();
    for (int i = 0; i < 3; ++i) {
        kernel_ms_mean[i] = launches ? (float)(sum[i] / (double)launches) : 0.0f;
        if (kernel_ms_min) kernel_ms_min[i] = low[i];
    }
    return rc;
}

int32_t kmx_lloyd_finalize(const kmx_lloyd_plan* plan, const void* centroids_t,
                           void* new_centroids_t, const void* cluster_sizes, void* workspace,
                           size_t workspace_bytes, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PLAN(plan);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(new_centroids_t);
    KMX_REQUIRE_PTR(cluster_sizes);
    KMX_REQUIRE_PTR(workspace);
    const int32_t d = plan->d, k = plan->k, dtype = plan->dtype;
    const LloydLayout L = lloyd_layout(plan->n, d, k, dtype, plan->flags);
    if (workspace_bytes < L.total) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    char* ws = (char*)workspace;
    auto* status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    double* shift_partial = reinterpret_cast<double*>(ws + L.off_shift);
    const unsigned grid = (unsigned)fin_grid(d, k);
#define KMX_FINALIZE(T, LANES)                                                                        \
    hipLaunchKernelGGL((lloyd_finalize_kernel<T, LANES>), dim3(grid), dim3(256), 0, stream,           \
                       (const T*)centroids_t, (T*)new_centroids_t, (const T*)cluster_sizes,           \
                       (T*)(ws + L.off_cpack), (T*)(ws + L.off_half), shift_partial, status, d, k,    \
                       L.dpad, 1)
    if (dtype == KMX_F32) {
        if (fin_lanes(d, k) == 64) KMX_FINALIZE(float, 64); else KMX_FINALIZE(float, 8);
    } else {
        if (fin_lanes(d, k) == 64) KMX_FINALIZE(double, 64); else KMX_FINALIZE(double, 8);
    }
#undef KMX_FINALIZE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_lloyd_status_read(const void* workspace, kmx_lloyd_status* status_host, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(workspace);
    KMX_REQUIRE_PTR(status_host);
    hipStream_t stream = (hipStream_t)stream_;
    hipError_t e = hipMemcpyAsync(status_host, workspace, sizeof(kmx_lloyd_status),
                                  hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) return (int32_t)e;
    e = hipStreamSynchronize(stream);
    return e == hipSuccess ? KMX_OK : (int32_t)e;
}

int32_t kmx_lloyd_recheck_count(const kmx_lloyd_plan* plan, const void* workspace,
                                uint32_t* count_host, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PLAN(plan);
    KMX_REQUIRE_PTR(workspace);
    KMX_REQUIRE_PTR(count_host);
    const int64_t n = plan->n;
    const int32_t d = plan->d, k = plan->k;
    const LloydLayout L = lloyd_layout(n, d, k, plan->dtype, plan->flags);
    *count_host = 0;
    const void* src = nullptr;
    if (L.screen || L.screen64)
        src = (const char*)workspace + L.off_bucket + sizeof(uint32_t);
    else if (L.variant == KMX_VARIANT_MFMA_WIDE && kmx_wide_screen_enabled(n, d, k, L.flags))
        src = kmx_wide_screen_counter((const char*)workspace + L.off_wscreen);
    else if (L.gemm_screen)
        src = kmx_gemm_screen_counter((const char*)workspace + L.off_wscreen);
    if (src == nullptr) return KMX_OK;
    hipStream_t stream = (hipStream_t)stream_;
    hipError_t e = hipMemcpyAsync(count_host, src, sizeof(uint32_t), hipMemcpyDeviceToHost, stream);
    if (e != hipSuccess) return (int32_t)e;
    e = hipStreamSynchronize(stream);
    return e == hipSuccess ? KMX_OK : (int32_t)e;
}

int32_t kmx_screen_scores(const void* X_t, const void* centroids_t, float* scores, float* bounds,
                          float* half_norms, float* scale, void* scratch, int64_t n, int32_t d,
                          int32_t k, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(scores);
    KMX_REQUIRE_PTR(bounds);
    KMX_REQUIRE_PTR(half_norms);
    KMX_REQUIRE_PTR(scale);
    KMX_REQUIRE_PTR(scratch);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    return kmx_screen_scores_impl((const float*)X_t, (const float*)centroids_t, scores, bounds, half_norms,
                                  scale, (unsigned int*)scratch, n, d, k, (hipStream_t)stream_);
}

size_t kmx_assign_workspace_bytes(int32_t d, int32_t k, int32_t dtype) {
    if (d <= 0 || k <= 0 || (dtype != KMX_F32 && dtype != KMX_F64)) return 0;
    return lloyd_layout(1, d, k, dtype, 0).off_bucket;
}

// Room for the screened tiled product behind the minimal workspace: max|c| per feature (the
// stand-in for max|x|), then the screen's header and list.
static size_t assign_gemm_screen_bytes(int64_t n, int d) {
    return kmx_align256((size_t)d * sizeof(unsigned int)) + kmx_gemm_screen_bytes(n);
}

size_t kmx_assign_workspace_bytes_for(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags) {
    const size_t base = kmx_assign_workspace_bytes(d, k, dtype);
    if (base == 0 || n <= 0 || dtype != KMX_F32 || !kmx_flags_valid(flags)) return base;
    const LloydLayout L = lloyd_layout(n, d, k, dtype, flags);
    if (L.gemm_screen) return kmx_align256(base) + assign_gemm_screen_bytes(n, d);
    if (L.variant != KMX_VARIANT_MFMA_WIDE) return base;
    const size_t extra = kmx_assign_wide_screen_bytes(n, d, k, flags);
    return extra ? kmx_align256(base) + extra : base;
}

int32_t kmx_assign_labels(const void* X_t, const void* centroids_t, uint32_t* labels,
                          void* workspace, size_t workspace_bytes, int64_t n, int32_t d, int32_t k,
                          int32_t dtype, uint32_t flags, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(workspace);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (!kmx_flags_valid(flags)) return KMX_ERR_BAD_ARGUMENT;
    LloydLayout L = lloyd_layout(n, d, k, dtype, flags);
    if (workspace_bytes < L.off_bucket) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    char* ws = (char*)workspace;
    if (dtype == KMX_F32) {
        // labels screened on the fp16 matrix cores: one kernel, straight from the centroids
        if (L.screen || L.screen_labels)
            return kmx_assign_labels_mfma_screen(X_t, centroids_t, labels, n, d, k, L.wgs_per_cu, stream);
        launch_pack<float>(centroids_t, ws + L.off_cpack, ws + L.off_half, nullptr, d, k, L.dpad, 0, 0.0, stream);
        KMX_LAUNCH_CHECK();
        if (L.variant == KMX_VARIANT_MFMA)
            return kmx_assign_labels_mfma_f32(L, X_t, centroids_t, labels, ws, n, d, k, stream);
        // few clusters on wide samples: the products of the labels on the matrix cores, straight from X_t
        if (L.variant == KMX_VARIANT_FEWK)
            return kmx_assign_labels_fewk(X_t, centroids_t, ws + L.off_half, labels, n, d, k, stream);
        if (L.variant == KMX_VARIANT_MFMA_WIDE) {
            // with the larger workspace of kmx_assign_workspace_bytes_for: labels screened in fp16
            const size_t extra = kmx_assign_wide_screen_bytes(n, d, k, flags);
            const size_t extra_off = kmx_align256(L.off_bucket);
            if (extra != 0 && workspace_bytes >= extra_off + extra)
                return kmx_assign_labels_wide_screen_f32(L, X_t, centroids_t, labels, ws, ws + extra_off, n, d,
                                                         k, stream);
            return kmx_assign_labels_mfma_wide_f32(L, X_t, centroids_t, labels, ws, n, d, k, stream);
        }
        // the tiled product screened in fp16 when the caller's workspace has room for its list
        // (kmx_assign_workspace_bytes_for); the scale then comes from the centroids
        const size_t extra_off = kmx_align256(L.off_bucket);
        unsigned int* absmax = nullptr;
        char* area = nullptr;
        if (L.gemm_screen && workspace_bytes >= extra_off + assign_gemm_screen_bytes(n, d)) {
            absmax = reinterpret_cast<unsigned int*>(ws + extra_off);
            area = ws + extra_off + kmx_align256((size_t)d * sizeof(unsigned int));
            const int32_t rc = kmx_wide_screen_scale_from_centroids(centroids_t, absmax, d, k, stream);
            if (rc != KMX_OK) return rc;
        }
        const int32_t rc = launch_fused<float, ACC_NONE>(L, X_t, nullptr, centroids_t,
                                                         (const float*)(ws + L.off_cpack),
                                                         (const float*)(ws + L.off_half), nullptr, labels, nullptr,
                                                         nullptr, n, d, k, stream, absmax, area);
        if (rc != KMX_OK) return rc;
    } else {
        // fp64 inputs of the screened step: the same kernel without the update
        if (L.screen64)
            return kmx_assign_labels_mfma_screen_f64(X_t, centroids_t, labels, n, d, k, L.wgs_per_cu, stream);
        launch_pack<double>(centroids_t, ws + L.off_cpack, ws + L.off_half, nullptr, d, k, L.dpad, 0, 0.0, stream);
        KMX_LAUNCH_CHECK();
        const int32_t rc = launch_fused<double, ACC_NONE>(L, X_t, nullptr, centroids_t,
                                                          (const double*)(ws + L.off_cpack),
                                                          (const double*)(ws + L.off_half), nullptr, labels, nullptr,
                                                          nullptr, n, d, k, stream);
        if (rc != KMX_OK) return rc;
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// Workspace of kmx_assign_labels_inertia: the label kernel's (with room for the wide path's list),
// then 8 fp64 partial sums per compute unit or what kmx_inertia wants, whichever is more.
static size_t assign_inertia_partials_bytes(int64_t n) {
    const size_t a = (size_t)kmx_num_cus() * 8 * sizeof(double);
    const size_t b = kmx_inertia_workspace_bytes(n);
    return kmx_align256(a > b ? a : b);
}

size_t kmx_assign_inertia_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags) {
    const size_t a = kmx_assign_workspace_bytes_for(n, d, k, dtype, flags);
    if (a == 0) return 0;
    return kmx_align256(a) + assign_inertia_partials_bytes(n);
}

int32_t kmx_assign_labels_inertia(const void* X_t, const void* sample_weight, const void* centroids_t,
                                  uint32_t* labels, void* out_total, void* workspace, size_t workspace_bytes,
                                  int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X_t);
    KMX_REQUIRE_PTR(centroids_t);
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(out_total);
    KMX_REQUIRE_PTR(workspace);
    if (n <= 0 || d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (!kmx_flags_valid(flags)) return KMX_ERR_BAD_ARGUMENT;
    const size_t need = kmx_assign_inertia_workspace_bytes(n, d, k, dtype, flags);
    if (need == 0 || workspace_bytes < need) return KMX_ERR_WORKSPACE;
    const size_t assign_bytes = kmx_align256(kmx_assign_workspace_bytes_for(n, d, k, dtype, flags));
    char* ws = (char*)workspace;
    double* partial = (double*)(ws + assign_bytes);
    hipStream_t stream = (hipStream_t)stream_;
    const LloydLayout L = lloyd_layout(n, d, k, dtype, flags);
    if (dtype == KMX_F32 && (L.screen || L.screen_labels)) {
        // one pass over X: the screened label kernel sums the inertia on the way
        int n_partials = 0;
        const int32_t rc = kmx_assign_labels_inertia_mfma_screen(X_t, sample_weight, centroids_t, labels, partial,
                                                                 &n_partials, n, d, k, L.wgs_per_cu, stream);
        if (rc != KMX_OK) return rc;
        return kmx_inertia_total_launch(partial, n_partials, out_total, dtype, stream);
    }
    const int32_t rc = kmx_assign_labels(X_t, centroids_t, labels, workspace, assign_bytes, n, d, k, dtype, flags, stream_);
    if (rc != KMX_OK) return rc;
    return kmx_inertia(X_t, sample_weight, centroids_t, labels, out_total, partial, assign_inertia_partials_bytes(n), n,
                       d, k, dtype, stream_);
}

}  // extern "C"
