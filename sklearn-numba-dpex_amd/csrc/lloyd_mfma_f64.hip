// fp64 fused Lloyd step on the matrix cores (gfx950), for d <= 64 when the (d + 1) * k
// accumulators and the centroids' operand fragments fit in the LDS of a compute unit.
//
// Replaces, for these shapes, the kernel pair fused_lloyd_single_step
// (sklearn_numba_dpex/kmeans/kernels/lloyd_single_step.py:35-424) + the zero-fill / half-norm
// helpers (common/kernels.py:38-57, 116-145); the reduction over the workgroups' partial sums
// and the finalisation stay with lloyd.hip.
//
//   * v_mfma_f64_16x16x4_f64: A = 16 centroids x 4 features (lane l: centroid l % 16, feature
//     l / 16), B = 4 features x 16 samples (lane l: feature l / 16, sample l % 16), D = 16 x 16
//     with lane l holding rows l / 16 + 4 r (r = 0..3) of column l % 16.
//   * A wave owns 64 consecutive samples: lane (g, j) = (l / 16, l % 16) loads the four samples
//     4 j .. 4 j + 3 of feature row 4 s + g with two 128-bit loads (a 16-lane group reads 512
//     contiguous bytes), and component t of that vector is the B operand of MFMA chain t, so
//     no shuffles.  Four independent chains per centroid block, accumulators start at
//     -0.5 ||c||^2, so after the K loop a lane holds <x, c> - 0.5 ||c||^2 for 4 centroids of
//     each of its 4 samples.
//   * fp64 MFMA and vector-ALU instructions do not overlap on this hardware (measured), so the
//     arg-max is kept short: per chain a 3-instruction max of the 4 rows, one compare, and only
//     the winning lanes copy the rows; the position is resolved once per tile.  Strict `>` in
//     increasing centroid order: the lowest index wins a tie.
//   * Partial sums in workgroup-private LDS accumulators (ds_add_f64 is fast on this part),
//     written to the workgroup's slot of `partial` at the end.
#include "lloyd_layout.h"

#include <type_traits>

namespace {

typedef double v4d __attribute__((ext_vector_type(4)));

// waves per workgroup (one workgroup per compute unit): two per SIMD with four sample columns
// per lane, three with two columns (fewer registers)
constexpr int f64_waves(int nc) { return nc == 2 ? 12 : 8; }

// NC (2 or 4) consecutive doubles of a row, as 128-bit loads.
template <int NC>
__device__ __forceinline__ void load_cols(const double* __restrict__ p, double (&v)[NC]) {
#pragma unroll
    for (int c = 0; c < NC; c += 2) {
        const double2 a = *reinterpret_cast<const double2*>(p + c);
        v[c] = a.x;
        v[c + 1] = a.y;
    }
}

// NC = sample columns per lane: a wave tile is 16 * NC samples and runs NC MFMA chains per
// centroid block.  NC = 2 leaves registers for the next tile's rows to be in flight during the
// current tile and for a third wave per SIMD.
template <int NKS, int NC, bool UPDATE>
__global__ __launch_bounds__(64 * f64_waves(NC)) void lloyd_mfma_f64_kernel(
    const double* __restrict__ X_t, const double* __restrict__ sample_weight,
    const double* __restrict__ centroids_t, const double* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    double* __restrict__ partial, kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k,
    int vec_ok) {
    if (status != nullptr && status->state != KMX_RUNNING) return;
    constexpr int F64_WAVES = f64_waves(NC);
    constexpr int THREADS = 64 * F64_WAVES;
    constexpr int TILE = 16 * NC;
    // (beyond 32 features the rows of one tile already take 64 registers)
    constexpr bool PREFETCH = NC == 2 && NKS <= 8;

    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int n_cb = (k + 15) >> 4;  // centroid blocks of 16
    const int items = (d + 1) * k;
    double* acc = reinterpret_cast<double*>(smem_raw);                   // [(d + 1) * k]
    double* afrag = acc + (UPDATE ? items : 0);                          // [n_cb][NKS][64]
    double* hneg = afrag + (size_t)n_cb * NKS * 64;                      // [n_cb * 16]
    __shared__ unsigned int changed_block;

    for (int idx = threadIdx.x; idx < n_cb * NKS * 64; idx += THREADS) {
        const int l = idx & 63;
        const int s = (idx >> 6) % NKS;
        const int cb = (idx >> 6) / NKS;
        const int c = 16 * cb + (l & 15);
        const int f = 4 * s + (l >> 4);
        afrag[idx] = (c < k && f < d) ? centroids_t[(size_t)f * k + c] : 0.0;
    }
    for (int c = threadIdx.x; c < n_cb * 16; c += THREADS)
        hneg[c] = c < k ? -half_norms[c] : -kmx_inf<double>();
    if (UPDATE) {
        for (int jx = threadIdx.x; jx < items; jx += THREADS) acc[jx] = 0.0;
        if (threadIdx.x == 0) changed_block = 0;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, j = lane & 15;
    const int64_t n_wtiles = (n + TILE - 1) / TILE;
    unsigned int changed = 0;

    // One tile: scores, arg-max, labels and (UPDATE) the accumulation.  FULL: every sample of
    // the tile exists and 128-bit accesses are legal.
    auto process = [&](auto full_tag, const double(&x)[NKS][NC], const double(&wv)[NC],
                       const uint32_t(&pl)[NC], const int64_t i0) {
        constexpr bool FULL = decltype(full_tag)::value;
        double best[NC];
        int code[NC];
        v4d sv[NC];  // the rows of the winning block
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            best[t] = -kmx_inf<double>();
            code[t] = 0;
            sv[t] = v4d{0.0, 0.0, 0.0, 0.0};
        }

        for (int cb = 0; cb < n_cb; ++cb) {
            const double* hp = hneg + cb * 16 + g;
            const v4d hv = {hp[0], hp[4], hp[8], hp[12]};
            const double* ap = afrag + (size_t)cb * NKS * 64 + lane;
            double af = ap[0];
            v4d a[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) a[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(af, x[0][t], hv, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < NKS; ++s) {
                af = ap[s * 64];
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    a[t] = __builtin_amdgcn_mfma_f64_16x16x4f64(af, x[s][t], a[t], 0, 0, 0);
            }
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                const double m = fmax(fmax(a[t][0], a[t][1]), fmax(a[t][2], a[t][3]));
                if (m > best[t]) {  // strict: the earlier block keeps a tie
                    best[t] = m;
                    code[t] = cb;
                    sv[t] = a[t];
                }
            }
        }

        // row inside the winning block (lowest row = lowest centroid of this lane), then the
        // four lane groups of a column are combined: highest score, lowest centroid on ties
        uint32_t lab[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            int pos = 3;
#pragma unroll
            for (int r = 2; r >= 0; --r) pos = (sv[t][r] == best[t]) ? r : pos;
            int c = 16 * code[t] + g + 4 * pos;
            double b = best[t];
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const double ob = __shfl_xor(b, off, 64);
                const int oc = __shfl_xor(c, off, 64);
                if (ob > b || (ob == b && oc < c)) {
                    b = ob;
                    c = oc;
                }
            }
            lab[t] = (uint32_t)c;
        }

        if (g == 0) {
            if constexpr (FULL && NC == 4) {
                *reinterpret_cast<uint4*>(labels + i0) = make_uint4(lab[0], lab[1], lab[2], lab[3]);
            } else if constexpr (FULL && NC == 2) {
                *reinterpret_cast<uint2*>(labels + i0) = make_uint2(lab[0], lab[1]);
            } else {
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    if (i0 + t < n) labels[i0 + t] = lab[t];
            }
        }

        if (UPDATE) {
            if (g == 0) {
#pragma unroll
                for (int t = 0; t < NC; ++t) {
                    changed += ((FULL || i0 + t < n) && pl[t] != lab[t]) ? 1u : 0u;
                    // samples past the end carry w = 0
                    if (FULL || i0 + t < n) kmx_atomic_add(acc + (size_t)d * k + lab[t], wv[t]);
                }
            }
#pragma unroll
            for (int s = 0; s < NKS; ++s) {
                const int f = 4 * s + g;
                if (f < d) {
                    double* rowacc = acc + (size_t)f * k;
#pragma unroll
                    for (int t = 0; t < NC; ++t)
                        if (FULL || i0 + t < n) kmx_atomic_add(rowacc + lab[t], x[s][t] * wv[t]);
                }
            }
        }
    };

    const int64_t wt_step = (int64_t)gridDim.x * F64_WAVES;
    const int64_t wt_first = (int64_t)blockIdx.x * F64_WAVES + wave;
    const int64_t n_fast = vec_ok ? n / TILE : 0;  // tiles entirely inside the array
    // rows 4 s + g of the lane's samples; a row past d - 1 reads row d - 1 (its A fragment is
    // zero and the update skips it), so that the loads are unconditional
    auto load_rows = [&](const int64_t wt, double(&dst)[NKS][NC]) {
        const double* __restrict__ p = X_t + wt * TILE + NC * j;
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
            const int f = 4 * s + g;
            load_cols<NC>(p + (size_t)(f < d ? f : d - 1) * n, dst[s]);
        }
    };
    if (wt_first < n_fast) {
        double xn[PREFETCH ? NKS : 1][NC];
        if constexpr (PREFETCH) load_rows(wt_first, xn);
        for (int64_t wt = wt_first; wt < n_fast; wt += wt_step) {
            const int64_t i0 = wt * TILE + NC * j;
            double x[NKS][NC];
            if constexpr (PREFETCH) {
#pragma unroll
                for (int s = 0; s < NKS; ++s)
#pragma unroll
                    for (int t = 0; t < NC; ++t) x[s][t] = xn[s][t];
                load_rows(wt + wt_step < n_fast ? wt + wt_step : wt, xn);
            } else {
                load_rows(wt, x);
            }
            double wv[NC];
            uint32_t pl[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                wv[t] = 0.0;
                pl[t] = 0u;
            }
            if (UPDATE) {
                load_cols<NC>(sample_weight + i0, wv);
                if constexpr (NC == 4) {
                    const uint4 p4 = *reinterpret_cast<const uint4*>(labels_prev + i0);
                    pl[0] = p4.x; pl[1] = p4.y; pl[2] = p4.z; pl[3] = p4.w;
                } else {
                    const uint2 p2 = *reinterpret_cast<const uint2*>(labels_prev + i0);
                    pl[0] = p2.x; pl[1] = p2.y;
                }
            }
            process(std::true_type{}, x, wv, pl, i0);
        }
    }
    // The rest: a partial last tile, or every tile when 128-bit accesses are not legal
    for (int64_t wt = n_fast + wt_first; wt < n_wtiles; wt += wt_step) {
        const int64_t i0 = wt * TILE + NC * j;
        double x[NKS][NC];
        double wv[NC];
        uint32_t pl[NC];
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
            const int f = 4 * s + g;
#pragma unroll
            for (int t = 0; t < NC; ++t)
                x[s][t] = (f < d && i0 + t < n) ? X_t[(size_t)f * n + i0 + t] : 0.0;
        }
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            wv[t] = 0.0;
            pl[t] = 0u;
            if (UPDATE && i0 + t < n) {
                wv[t] = sample_weight[i0 + t];
                pl[t] = labels_prev[i0 + t];
            }
        }
        process(std::false_type{}, x, wv, pl, i0);
    }

    if (UPDATE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        double* out = partial + (size_t)blockIdx.x * items;
        for (int jx = threadIdx.x; jx < items; jx += THREADS) out[jx] = acc[jx];
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
    }
}

size_t mfma_f64_lds_bytes(int d, int k, bool update) {
    const int nks = (d + 3) / 4, n_cb = (k + 15) / 16;
    size_t bytes = ((size_t)n_cb * nks * 64 + (size_t)n_cb * 16) * sizeof(double);
    if (update) bytes += (size_t)(d + 1) * k * sizeof(double);
    return bytes;
}

}  // namespace

// One workgroup per compute unit may take all of its LDS (160 KB less the static variables).
bool kmx_mfma_f64_supported(int d, int k) {
    return d <= 64 && k >= 16 && mfma_f64_lds_bytes(d, k, true) <= 160 * 1024 - 256;
}

bool kmx_mfma_f64_labels_supported(int d, int k) {
    return d <= 64 && k >= 16 && mfma_f64_lds_bytes(d, k, false) <= 160 * 1024 - 256;
}

// Sample columns per lane: two (three waves per SIMD, next tile in flight) once there are
// several tiles per wave, four for small inputs.  KMX_FLAG_COLS(2 | 4) overrides this for
// experiments.  More than 32 features: two (four would need 128 registers for the rows).
static int f64_cols(int64_t n, int d, int cols) {
    if (d > 32) return 2;
    if (cols == 2 || cols == 4) return cols;
    return n >= (int64_t)1 << 19 ? 2 : 4;
}

int kmx_mfma_f64_grid(int64_t n, int d, int wgs_per_cu, int cols_asked, int max_slots) {
    const int nc = f64_cols(n, d, cols_asked);
    const int64_t tiles = kmx_cdiv(kmx_cdiv(n, 16 * nc), f64_waves(nc));
    const int64_t cap = (int64_t)(wgs_per_cu > 0 ? wgs_per_cu : 1) * kmx_num_cus();
    int64_t grid = tiles < cap ? tiles : cap;
    if (grid > max_slots) grid = max_slots;
    return grid < 1 ? 1 : (int)grid;
}

int32_t kmx_lloyd_step_mfma_f64(const void* X_t, const void* w, const void* centroids_t,
                                const void* half_norms, const uint32_t* labels_prev,
                                uint32_t* labels, void* partial, kmx_lloyd_status* status,
                                int64_t n, int d, int k, bool update, int wgs_per_cu, int cols_asked,
                                int max_slots, hipStream_t stream) {
    if (!(update ? kmx_mfma_f64_supported(d, k) : kmx_mfma_f64_labels_supported(d, k)))
        return KMX_ERR_UNSUPPORTED;
    const size_t lds = mfma_f64_lds_bytes(d, k, update);
    const int grid = kmx_mfma_f64_grid(n, d, wgs_per_cu, cols_asked, max_slots);
    auto aligned16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    // rows start 16-byte aligned when n is even; 4 samples per lane need n % 4 == 0 only for
    // the 128-bit label accesses
    const int vec_ok = (n % 4 == 0) && aligned16(X_t) && aligned16(labels) &&
                       (!update || (aligned16(w) && aligned16(labels_prev)));
    const int cols = f64_cols(n, d, cols_asked);
#define KMX_F64_LAUNCH(NKS, NC, UPD)                                                              \
    if (lds > 64 * 1024) {                                                                        \
        const hipError_t e = hipFuncSetAttribute(                                                 \
            reinterpret_cast<const void*>(&lloyd_mfma_f64_kernel<NKS, NC, UPD>),                   \
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                \
        if (e != hipSuccess) return (int32_t)e;                                                   \
    }                                                                                             \
    hipLaunchKernelGGL((lloyd_mfma_f64_kernel<NKS, NC, UPD>), dim3((unsigned)grid),                 \
                       dim3(64 * f64_waves(NC)), lds, stream, (const double*)X_t, (const double*)w, \
                       (const double*)centroids_t, (const double*)half_norms, labels_prev, labels,  \
                       (double*)partial, status, n, d, k, vec_ok)
#define KMX_F64_CASE(NKS)                                    \
    do {                                                     \
        if (cols == 2) {                                     \
            if (update) { KMX_F64_LAUNCH(NKS, 2, true); }    \
            else { KMX_F64_LAUNCH(NKS, 2, false); }          \
        } else {                                             \
            if (update) { KMX_F64_LAUNCH(NKS, 4, true); }    \
            else { KMX_F64_LAUNCH(NKS, 4, false); }          \
        }                                                    \
    } while (0)
    switch ((d + 3) / 4) {
        case 1: KMX_F64_CASE(1); break;
        case 2: KMX_F64_CASE(2); break;
        case 3: KMX_F64_CASE(3); break;
        case 4: KMX_F64_CASE(4); break;
        case 5: KMX_F64_CASE(5); break;
        case 6: KMX_F64_CASE(6); break;
        case 7: KMX_F64_CASE(7); break;
        case 8: KMX_F64_CASE(8); break;
#define KMX_F64_CASE2(NKS)                            \
    do {                                              \
        if (update) { KMX_F64_LAUNCH(NKS, 2, true); } \
        else { KMX_F64_LAUNCH(NKS, 2, false); }       \
    } while (0)
        case 9: KMX_F64_CASE2(9); break;
        case 10: KMX_F64_CASE2(10); break;
        case 11: KMX_F64_CASE2(11); break;
        case 12: KMX_F64_CASE2(12); break;
        case 13: KMX_F64_CASE2(13); break;
        case 14: KMX_F64_CASE2(14); break;
        case 15: KMX_F64_CASE2(15); break;
        default: KMX_F64_CASE2(16); break;
#undef KMX_F64_CASE2
    }
#undef KMX_F64_LAUNCH
#undef KMX_F64_CASE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
