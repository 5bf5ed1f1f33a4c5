// fp32 fused Lloyd step on the matrix cores of gfx950 (v_mfma_f32_32x32x2_f32), one launch
// per iteration.
//
// Work decomposition
//   * A wave owns tiles of 32 * MC consecutive samples, MC = 2 or 4 sample columns per lane.
//     Lane (j, h) with j = lane % 32, h = lane / 32 loads, for every pair of features
//     (2s, 2s + 1), the samples MC j .. MC j + MC - 1 of feature row 2s + h with one 64- or
//     128-bit load: each half-wave reads 256 or 512 contiguous bytes of X_t.  Component t of
//     that vector is exactly the B operand (K x N = 2 x 32) of MFMA chain t, which holds the
//     samples {MC j + t}; no shuffles.
//   * Centroids are the A operand (M x K = 32 x 2), staged once per workgroup in LDS in
//     fragment order (conflict-free 4-byte reads, one per MFMA), 32 centroids per block.
//   * The accumulator of tile t starts at -0.5||c||^2, so after the K loop it holds
//     <x, c> - 0.5||c||^2 for 16 centroids x 1 sample per lane and chain; the argmax over centroids is
//     kept per lane in registers (strict '>' in increasing centroid order = lowest index
//     wins) and the two half-waves are combined once per tile.
//   * w * x and w are accumulated in 64-bit FIXED POINT: LDS accumulators private to the
//     workgroup (ds_add_u64 runs ~10x faster than ds_add_f32 on this hardware), flushed once
//     per workgroup with 64-bit integer global atomics.  Integer addition is associative, so
//     the sums do not depend on the order in which samples, waves or workgroups arrive: the
//     iteration is reproducible bit for bit, and the sums are exact to 2^-q (q chosen per
//     feature from max|x|, max|w| and n so that nothing can overflow).
//   * A one-workgroup kernel then converts the sums, lists empty clusters and, if there are
//     none, divides, computes the shift and runs the convergence test (lloyd_tail.h).
//
// Arithmetic per sample is the reference's 0.5||c||^2 - <x, c> with another summation
// order, so labels can differ from a feature-sequential evaluation only at near-ties.
#include "lloyd_layout.h"
#include "lloyd_tail.h"

#include <type_traits>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v8d __attribute__((ext_vector_type(8)));

// 1.5 * 2^52: adding it to |v| < 2^51 leaves round-to-nearest(v) in the low mantissa bits.
constexpr double FIX_MAGIC = 6755399441055744.0;
constexpr long long FIX_MAGIC_BITS = 0x4338000000000000ll;

__device__ __forceinline__ unsigned long long to_fixed(double scaled_plus_magic) {
    return (unsigned long long)(__double_as_longlong(scaled_plus_magic) - FIX_MAGIC_BITS);
}

// ---------------------------------------------------------------------------- scales

__global__ void absmax_zero_kernel(unsigned int* absmax, int count) {
    for (int i = threadIdx.x; i < count; i += blockDim.x) absmax[i] = 0u;
}

// Row r < d: max |X_t[r, :]|; row d: max |w|.  Non-negative floats order like their bits.
// (fp64 inputs: the maximum of the values rounded to fp32, which is what the screened step works
// with; its fixed-point exponents leave a factor of two of room above it)
__device__ __forceinline__ float amax_vec(float a, const float4& v) {
    return fmaxf(fmaxf(a, fabsf(v.x)), fmaxf(fabsf(v.y), fmaxf(fabsf(v.z), fabsf(v.w))));
}
__device__ __forceinline__ float amax_vec(float a, const double2& v) {
    return fmaxf(a, fmaxf(fabsf((float)v.x), fabsf((float)v.y)));
}
template <typename T>
__global__ __launch_bounds__(256) void absmax_rows_kernel(const T* __restrict__ X_t,
                                                          const T* __restrict__ w,
                                                          unsigned int* __restrict__ absmax,
                                                          int64_t n, int d, int vec_ok) {
    const int row = blockIdx.y;
    const T* __restrict__ p = row < d ? X_t + (size_t)row * n : w;
    float m = 0.0f;
    const int64_t stride = (int64_t)gridDim.x * 256;
    if (vec_ok) {
        // rows start 16-byte aligned and n is a multiple of 4: 128-bit loads
        using V = std::conditional_t<sizeof(T) == 8, double2, float4>;
        const V* __restrict__ p4 = reinterpret_cast<const V*>(p);
        const int64_t n4 = n / (int64_t)(16 / sizeof(T));
        int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
        for (; g + 3 * stride < n4; g += 4 * stride) {  // four loads in flight per lane
            const V v0 = p4[g], v1 = p4[g + stride], v2 = p4[g + 2 * stride], v3 = p4[g + 3 * stride];
            m = amax_vec(amax_vec(amax_vec(amax_vec(m, v0), v1), v2), v3);
        }
        for (; g < n4; g += stride) m = amax_vec(m, p4[g]);
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
            m = fmaxf(m, fabsf((float)p[i]));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    // one atomic per workgroup: thousands of waves on the same few words serialise in L2
    __shared__ float wave_max[4];
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
        atomicMax(&absmax[row], __float_as_uint(m));
    }
}

// q[f] for the sums of w * x_f, q[d] for the sums of w: the largest exponents such that
// n * max|w| * max|x_f| * 2^q < 2^61 and one sample's contribution stays below 2^50.
__global__ void fixed_point_exponents_kernel(const unsigned int* __restrict__ absmax,
                                             int* __restrict__ q, int64_t n, int d) {
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    if (f > d) return;
    const float wmax = __uint_as_float(absmax[d]);
    const float xmax = f < d ? __uint_as_float(absmax[f]) : 1.0f;
    int e = 0;  // log2 upper bound of one contribution
    if (wmax > 0.0f && isfinite(wmax)) e += ilogbf(wmax) + 1;
    if (f < d && xmax > 0.0f && isfinite(xmax)) e += ilogbf(xmax) + 1;
    int en = 1;
    while (((int64_t)1 << en) < n && en < 62) ++en;  // n <= 2^en
    int qv = 61 - (e + en);
    if (qv > 50 - e) qv = 50 - e;
    if (qv > 100) qv = 100;
    if (qv < -100) qv = -100;
    q[f] = qv;
}

// ---------------------------------------------------------------------------- fused step

// NKS = K steps held in registers.  EXACT: the shape has exactly NKS steps, so the K loop has
// no guards and the body of the centroid-block loop is one basic block (the scheduler can
// hoist the LDS reads of the A fragments above the MFMAs); otherwise steps s >= nks are
// skipped with wave-uniform branches.
constexpr int ARGMAX_GROUP = 8;  // accumulator registers per argmax group: 2, 4, 8 or 16

// Waves per workgroup: with few K steps the kernel fits two (four sample columns per lane) or
// three (two columns) waves per SIMD, and ONE workgroup per compute unit keeps the accumulator
// flushes (the global atomics of all workgroups hit the same (d + 1) * k addresses) and the
// staging work at their minimum.
#ifndef KMX_MC2_WAVES
#define KMX_MC2_WAVES 12
#endif
constexpr int mfma_waves(int nks, int mc) { return nks <= 8 ? (mc == 2 ? KMX_MC2_WAVES : 8) : 4; }

template <int NKS, bool EXACT, bool UPDATE, int MC>
__global__ __launch_bounds__(64 * mfma_waves(NKS, MC)) void lloyd_mfma_kernel(
    const float* __restrict__ X_t, const float* __restrict__ sample_weight,
    const float* __restrict__ centroids_t, const uint32_t* __restrict__ labels_prev,
    uint32_t* __restrict__ labels, kmx_lloyd_status* __restrict__ status,
    const int* __restrict__ q_exp, unsigned long long* __restrict__ gsum, int64_t n, int d, int k,
    int vec_ok) {
    if (UPDATE && status->state != KMX_RUNNING) return;

    constexpr int WAVES = mfma_waves(NKS, MC), THREADS = 64 * WAVES;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int nks = EXACT ? NKS : (d + 1) >> 1;  // K steps of 2 features
    const int n_cb = (k + 31) >> 5;        // centroid blocks of 32
    const int items = (d + 1) * k;
    unsigned long long* acc = reinterpret_cast<unsigned long long*>(smem_raw);  // [(d + 1) * k]
    float* afrag = reinterpret_cast<float*>(acc + (UPDATE ? items : 0));         // [n_cb][nks][64]
    float* hneg = afrag + n_cb * nks * 64;  // [n_cb][2][16]  -0.5||c||^2 in accumulator order
    float* qscale = hneg + n_cb * 32;       // [d + 1]  2^q of the fixed-point sums (UPDATE)
    __shared__ unsigned int changed_block;

    for (int idx = threadIdx.x; idx < n_cb * nks * 64; idx += THREADS) {
        const int l = idx & 63;
        const int s = (idx >> 6) % nks;
        const int cb = (idx >> 6) / nks;
        const int c = 32 * cb + (l & 31);
        const int f = 2 * s + (l >> 5);
        afrag[idx] = (c < k && f < d) ? centroids_t[(size_t)f * k + c] : 0.0f;
    }
    for (int idx = threadIdx.x; idx < n_cb * 32; idx += THREADS) {
        const int cb = idx >> 5, h = (idx >> 4) & 1, r = idx & 15;
        const int c = 32 * cb + 8 * (r >> 2) + 4 * h + (r & 3);
        float v = -kmx_inf<float>();
        if (c < k) {
            float sq = 0.0f;
            for (int f = 0; f < d; ++f) {
                const float cv = centroids_t[(size_t)f * k + c];
                sq += cv * cv;
            }
            v = -(sq / 2.0f);
        }
        hneg[idx] = v;
    }
    if (UPDATE) {
        for (int jx = threadIdx.x; jx < items; jx += THREADS) acc[jx] = 0ull;
        for (int f = threadIdx.x; f <= d; f += THREADS) qscale[f] = ldexpf(1.0f, q_exp[f]);
        if (threadIdx.x == 0) changed_block = 0;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int64_t n_wtiles = (n + 32 * MC - 1) / (32 * MC);
    unsigned int changed = 0;

    // 2^q of the feature rows this lane accumulates (row 2s + h), and of the weights
    float scale[NKS];
    float scale_w = 1.0f;
    if (UPDATE) {
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
            const int f = 2 * s + h;
            scale[s] = (s < nks && f < d) ? qscale[f] : 0.0f;
        }
        scale_w = qscale[d];
    }

    // One tile of NC sample columns per lane: scores on the matrix cores, argmax, labels and
    // (UPDATE) the accumulation.  NC = 4: 128 samples, the lane's samples are i0 .. i0 + 3;
    // NC = 1: 32 samples (a quarter tile), the lane's sample is i0.  FULL: every sample of the
    // tile exists and (NC = 4) 128-bit accesses are legal.  wv / pl: weights and previous
    // labels of the lane's samples.
    // +inf the optimiser cannot see through (it would turn the median in the arg-max into a
    // maximum with two canonicalising instructions in front)
    float pos_inf = kmx_inf<float>();
    asm volatile("" : "+s"(pos_inf));
    auto process = [&](auto nc_tag, auto full_tag, const float(&x)[NKS][decltype(nc_tag)::value],
                       const float(&wv)[decltype(nc_tag)::value],
                       const uint32_t(&pl)[decltype(nc_tag)::value], const int64_t i0) {
        constexpr int NC = decltype(nc_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;
        // Running argmax per sample column, by groups of ARGMAX_GROUP accumulator registers:
        // a group costs one max chain, one compare and the conditional copies of its values
        // (about 1.4 VALU instructions per score instead of 3 for a compare and two selects
        // per score; fp32 MFMA and VALU instructions do not overlap on this hardware, so every
        // VALU instruction saved is time saved).  The position inside the winning group is
        // found once per tile.
        float best[NC];
        int code[NC];
        double svd[NC][ARGMAX_GROUP / 2];  // the winning group's registers, as pairs
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            best[t] = -kmx_inf<float>();
            code[t] = 0;
#pragma unroll
            for (int r = 0; r < ARGMAX_GROUP / 2; ++r) svd[t][r] = 0.0;
        }

        for (int cb = 0; cb < n_cb; ++cb) {
            const float* hp = hneg + cb * 32 + h * 16;
            v16f hv;
#pragma unroll
            for (int r = 0; r < 16; ++r) hv[r] = hp[r];
            const float* ap = afrag + (size_t)cb * nks * 64 + lane;
            // the first K step reads the accumulator start (-0.5||c||^2) straight from hv
            float af = ap[0];
            v16f a[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) a[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(af, x[0][t], hv, 0, 0, 0);
#pragma unroll
            for (int s = 1; s < NKS; ++s) {
                if (s < nks) {
                    af = ap[s * 64];
#pragma unroll
                    for (int t = 0; t < NC; ++t)
                        a[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(af, x[s][t], a[t], 0, 0, 0);
                }
            }
#pragma unroll
            for (int g = 0; g < 16 / ARGMAX_GROUP; ++g) {
                const int cd = cb * (16 / ARGMAX_GROUP) + g;  // wave-uniform
#pragma unroll
                for (int t = 0; t < NC; ++t) {
                    // three-operand max: two scores per instruction (fmaxf would also
                    // canonicalise the matrix-core results first).  The FIRST read of a
                    // matrix-core result must be an instruction the compiler knows (the median
                    // of a, b and +inf is max(a, b)): it inserts the wait states an MFMA result
                    // needs before a vector-ALU read, which it does not do for operands of
                    // inline assembly.  Once that instruction has issued the whole MFMA is
                    // complete, so the rest of the chain may be assembly.
                    static_assert(ARGMAX_GROUP % 2 == 0, "pairs of registers");
                    float m = __builtin_amdgcn_fmed3f(a[t][g * ARGMAX_GROUP], a[t][g * ARGMAX_GROUP + 1], pos_inf);
#pragma unroll
                    for (int r = 2; r + 1 < ARGMAX_GROUP; r += 2)
                        asm("v_max3_f32 %0, %1, %2, %3"
                            : "=v"(m)
                            : "v"(m), "v"(a[t][g * ARGMAX_GROUP + r]), "v"(a[t][g * ARGMAX_GROUP + r + 1]));
                    // strict: the earlier group keeps a tie.  The winning lanes copy the
                    // group with 64-bit moves under the execution mask: half the instructions
                    // of per-register selects.
                    if (m > best[t]) {
                        best[t] = m;
                        code[t] = cd;
                        const v8d ad = __builtin_bit_cast(v8d, a[t]);
#pragma unroll
                        for (int r = 0; r < ARGMAX_GROUP / 2; ++r)
                            asm volatile("v_mov_b64 %0, %1"
                                         : "+v"(svd[t][r])
                                         : "v"(ad[g * (ARGMAX_GROUP / 2) + r]));
                    }
                }
            }
        }

        // position inside the winning group (lowest register = lowest centroid of this lane),
        // (block, register) -> centroid index, then combine the two half-waves
        uint32_t lab[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            float sv[ARGMAX_GROUP];
#pragma unroll
            for (int r = 0; r < ARGMAX_GROUP / 2; ++r) {
                const float2 pr = __builtin_bit_cast(float2, svd[t][r]);
                sv[2 * r] = pr.x;
                sv[2 * r + 1] = pr.y;
            }
            int pos = ARGMAX_GROUP - 1;
#pragma unroll
            for (int r = ARGMAX_GROUP - 2; r >= 0; --r) pos = (sv[r] == best[t]) ? r : pos;
            const int reg = (code[t] % (16 / ARGMAX_GROUP)) * ARGMAX_GROUP + pos;
            const int blk = code[t] / (16 / ARGMAX_GROUP);
            int c = 32 * blk + 8 * (reg >> 2) + 4 * h + (reg & 3);
            const float ov = __shfl_xor(best[t], 32, 64);
            const int oc = __shfl_xor(c, 32, 64);
            if (ov > best[t] || (ov == best[t] && oc < c)) c = oc;
            lab[t] = (uint32_t)c;
        }

        if (h == 0) {
            if constexpr (FULL && NC == 4) {
                *reinterpret_cast<uint4*>(labels + i0) = make_uint4(lab[0], lab[1], lab[2], lab[3]);
            } else if constexpr (FULL && NC == 2) {
                *reinterpret_cast<uint2*>(labels + i0) = make_uint2(lab[0], lab[1]);
            } else {
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    if (FULL || i0 + t < n) labels[i0 + t] = lab[t];
            }
        }

        if (UPDATE) {
            if (h == 0) {
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    changed += ((FULL || i0 + t < n) && pl[t] != lab[t]) ? 1u : 0u;
            }
            // samples past the end carry w = 0 and x = 0: they add zero
            double wd[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) wd[t] = (double)wv[t];
#pragma unroll
            for (int s = 0; s < NKS; ++s) {
                const int f = 2 * s + h;
                if (s < nks && f < d) {
                    unsigned long long* rowacc = acc + f * k;
                    const double sc = (double)scale[s];
#pragma unroll
                    for (int t = 0; t < NC; ++t) {
                        // x * w is exact in fp64; one rounding, to a multiple of 2^-q
                        const double v = fma((double)x[s][t], wd[t] * sc, FIX_MAGIC);
                        atomicAdd(rowacc + lab[t], to_fixed(v));
                    }
                }
            }
            if (h == 0) {
                unsigned long long* szacc = acc + d * k;
                const double sc = (double)scale_w;
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    atomicAdd(szacc + lab[t], to_fixed(fma(wd[t], sc, FIX_MAGIC)));
            }
        }
    };
    using ColsM = std::integral_constant<int, MC>;
    using Cols1 = std::integral_constant<int, 1>;
    constexpr int TILE = 32 * MC;  // samples of a full wave tile

    const int64_t wt_step = (int64_t)gridDim.x * WAVES;
    const int64_t wt_first = (int64_t)blockIdx.x * WAVES + wave;
    // Tiles that lie entirely inside the array, when vector accesses are legal: straight-line
    // loads with the next tile's rows in flight during the current tile (the wave does not
    // stall on its own loads or on the completion of its label store).
    const int64_t n_fast = vec_ok ? n / TILE : 0;
    // The last round of full tiles would keep only n_fast % wt_step of the waves busy for a
    // whole tile time.  When it is at most three quarters full it is cut into single-column
    // tiles of 32 samples instead (one MFMA chain per wave), spread over all the waves.
    const int64_t n_rounds = n_fast / wt_step;
    const int64_t n_left = n_fast - n_rounds * wt_step;
    const bool quarters = MC > 1 && n_left > 0 && 4 * n_left <= 3 * wt_step;
    const int64_t n_main = quarters ? n_rounds * wt_step : n_fast;
    // Rows of the lane's half-wave (2s + h) at the lane's MC samples.  The loads are
    // unconditional, so that the compiler can count them exactly and wait for the older tile
    // only: a row past d - 1 (odd d, upper half-wave, last K step) reads row d - 1 instead;
    // its A fragment is zero and the accumulation skips it.
    const float* __restrict__ xrow_base = X_t + (size_t)h * n + MC * j;
    const int last_row = 2 * (nks - 1) + h < d ? 2 * (nks - 1) + h : d - 1;
    const size_t last_row_off = (size_t)(last_row - h) * n;
    auto load_cols = [&](const float* __restrict__ p, float(&v)[MC]) {
        if constexpr (MC == 4) {
            const float4 q = *reinterpret_cast<const float4*>(p);
            v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
            const float2 q = *reinterpret_cast<const float2*>(p);
            v[0] = q.x; v[1] = q.y;
        }
    };
    auto load_rows = [&](const int64_t wt, float(&dst)[NKS][MC]) {
        const float* __restrict__ p = xrow_base + wt * TILE;
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
            if (EXACT || s < nks) {
                const size_t off = (s == nks - 1) ? last_row_off : (size_t)(2 * s) * n;
                load_cols(p + off, dst[s]);
            } else {
#pragma unroll
                for (int t = 0; t < MC; ++t) dst[s][t] = 0.0f;
            }
        }
    };
    constexpr bool PREFETCH = NKS <= 16;  // the double buffer costs MC * NKS registers
    if (wt_first < n_main) {
        float xn[PREFETCH ? NKS : 1][MC];
        if constexpr (PREFETCH) load_rows(wt_first, xn);
        for (int64_t wt = wt_first; wt < n_main; wt += wt_step) {
            const int64_t i0 = wt * TILE + MC * j;
            float x[NKS][MC];
            if constexpr (PREFETCH) {
#pragma unroll
                for (int s = 0; s < NKS; ++s)
#pragma unroll
                    for (int t = 0; t < MC; ++t) x[s][t] = xn[s][t];
                // past the last tile the same rows are read again (and not used)
                load_rows(wt + wt_step < n_main ? wt + wt_step : wt, xn);
            } else {
                load_rows(wt, x);
            }
            float wv[MC];
            uint32_t pl[MC];
#pragma unroll
            for (int t = 0; t < MC; ++t) {
                wv[t] = 0.f;
                pl[t] = 0u;
            }
            if (UPDATE) {
                load_cols(sample_weight + i0, wv);
                if constexpr (MC == 4) {
                    const uint4 p4 = *reinterpret_cast<const uint4*>(labels_prev + i0);
                    pl[0] = p4.x; pl[1] = p4.y; pl[2] = p4.z; pl[3] = p4.w;
                } else {
                    const uint2 p2 = *reinterpret_cast<const uint2*>(labels_prev + i0);
                    pl[0] = p2.x; pl[1] = p2.y;
                }
            }
            process(ColsM{}, std::true_type{}, x, wv, pl, i0);
        }
    }
    if (quarters) {
        // single-column tile q of the left-over tiles: samples [n_main * TILE + 32 q, + 32),
        // lane j takes sample j of it (128 contiguous bytes per half-wave and row)
        for (int64_t q = wt_first; q < MC * n_left; q += wt_step) {
            const int64_t i0 = n_main * TILE + 32 * q + j;
            float x[NKS][1];
#pragma unroll
            for (int s = 0; s < NKS; ++s) {
                const int f = 2 * s + h;
                x[s][0] = (s < nks && f < d) ? X_t[(size_t)f * n + i0] : 0.0f;
            }
            float wv[1] = {0.f};
            uint32_t pl[1] = {0u};
            if (UPDATE) {
                wv[0] = sample_weight[i0];
                pl[0] = labels_prev[i0];
            }
            process(Cols1{}, std::true_type{}, x, wv, pl, i0);
        }
    }
    // The rest: a partial last tile, or every tile when vector accesses are not legal
    for (int64_t wt = n_fast + wt_first; wt < n_wtiles; wt += wt_step) {
        const int64_t i0 = wt * TILE + MC * j;
        float x[NKS][MC];
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
            const int f = 2 * s + h;
#pragma unroll
            for (int t = 0; t < MC; ++t)
                x[s][t] = (s < nks && f < d && i0 + t < n) ? X_t[(size_t)f * n + i0 + t] : 0.0f;
        }
        float wv[MC];
        uint32_t pl[MC];
#pragma unroll
        for (int t = 0; t < MC; ++t) {
            wv[t] = 0.f;
            pl[t] = 0u;
            if (UPDATE && i0 + t < n) {
                wv[t] = sample_weight[i0 + t];
                pl[t] = labels_prev[i0 + t];
            }
        }
        process(ColsM{}, std::false_type{}, x, wv, pl, i0);
    }

    if (UPDATE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
        for (int jx = threadIdx.x; jx < items; jx += THREADS) {
            const unsigned long long v = acc[jx];
            if (v) atomicAdd(gsum + jx, v);
        }
    }
}

size_t mfma_lds_bytes(int d, int k, bool update) {
    const int nks = (d + 1) / 2, n_cb = (k + 31) / 32;
    size_t bytes = ((size_t)n_cb * nks * 64 + (size_t)n_cb * 32) * sizeof(float);
    if (update) bytes += (size_t)(d + 1) * k * sizeof(unsigned long long) + (size_t)(d + 1) * sizeof(float);
    return bytes;
}

template <bool UPDATE>
int32_t launch_mfma(const LloydLayout& L, const void* X_t, const void* w, const void* centroids_t,
                    const uint32_t* labels_prev, uint32_t* labels, kmx_lloyd_status* status,
                    const int* q_exp, unsigned long long* gsum, int64_t n, int d, int k,
                    hipStream_t stream) {
    const size_t lds = mfma_lds_bytes(d, k, UPDATE);
    if (lds > 64 * 1024 || d > 64) return KMX_ERR_UNSUPPORTED;
    const int nks_t = (d + 1) / 2 <= 8 ? (d + 1) / 2 : (d <= 32 ? 16 : 32);
    // Sample columns per lane.  Two (64 samples per wave tile, two MFMA chains) leave
    // registers for three waves per SIMD and run about 4 % faster than four columns with two
    // waves; KMX_FLAG_COLS(4) restores the latter for experiments.  Shapes with more than 8 K
    // steps keep four columns and four waves per workgroup.
    const int mc = (nks_t <= 8 && L.cols != 4) ? 2 : 4;
    const int64_t n_wtiles = kmx_cdiv(n, 32 * mc);
    const int waves = mfma_waves(nks_t, mc);
    int64_t grid = kmx_cdiv(n_wtiles, waves);
    // resident workgroups only: one workgroup per compute unit, or two of four waves
    const int per_cu = waves >= 8 ? 1 : 2;
    const int cap = (L.wgs_per_cu > 0 ? L.wgs_per_cu : per_cu) * kmx_num_cus();
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
    auto aligned16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    const int vec_ok = (n % 4 == 0) && aligned16(X_t) && aligned16(labels) &&
                       (!UPDATE || (aligned16(w) && aligned16(labels_prev)));
#define KMX_MFMA_LAUNCH(NKS, EXACT, MC)                                                           \
    hipLaunchKernelGGL((lloyd_mfma_kernel<NKS, EXACT, UPDATE, MC>), dim3((unsigned)grid),          \
                       dim3(64 * mfma_waves(NKS, MC)), lds, stream, (const float*)X_t,             \
                       (const float*)w, (const float*)centroids_t, labels_prev, labels, status,    \
                       q_exp, gsum, n, d, k, vec_ok)
#define KMX_MFMA_CASE(NKS, EXACT)                    \
    do {                                             \
        if (mc == 2 && NKS <= 8)                     \
            KMX_MFMA_LAUNCH(NKS, EXACT, 2);          \
        else                                         \
            KMX_MFMA_LAUNCH(NKS, EXACT, 4);          \
    } while (0)
    switch ((d + 1) / 2) {
        case 1: KMX_MFMA_CASE(1, true); break;
        case 2: KMX_MFMA_CASE(2, true); break;
        case 3: KMX_MFMA_CASE(3, true); break;
        case 4: KMX_MFMA_CASE(4, true); break;
        case 5: KMX_MFMA_CASE(5, true); break;
        case 6: KMX_MFMA_CASE(6, true); break;
        case 7: KMX_MFMA_CASE(7, true); break;
        case 8: KMX_MFMA_CASE(8, true); break;
        default:
            if (d <= 32)
                KMX_MFMA_CASE(16, false);
            else
                KMX_MFMA_CASE(32, false);
    }
#undef KMX_MFMA_CASE
#undef KMX_MFMA_LAUNCH
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

}  // namespace

bool kmx_mfma_supported(int d, int k) {
    return d <= 64 && k >= 16 && mfma_lds_bytes(d, k, true) <= 64 * 1024;
}

int32_t kmx_lloyd_mfma_prepare(const LloydLayout& L, const void* X_t, const void* w, char* ws,
                               int64_t n, int d, int dtype, hipStream_t stream) {
    unsigned int* absmax = reinterpret_cast<unsigned int*>(ws + L.off_scales);
    int* q_exp = reinterpret_cast<int*>(absmax + (d + 1));
    hipLaunchKernelGGL(absmax_zero_kernel, dim3(1), dim3(256), 0, stream, absmax, d + 1);
    int64_t gx = kmx_cdiv(n, 256 * 64);
    if (gx > 64) gx = 64;
    if (gx * (d + 1) < 1024) gx = kmx_cdiv(1024, d + 1) < kmx_cdiv(n, 1024) ? kmx_cdiv(1024, d + 1) : kmx_cdiv(n, 1024);
    const int vec_ok = (n % 4 == 0) && ((((uintptr_t)X_t) & 15) == 0) && ((((uintptr_t)w) & 15) == 0);
    if (dtype == KMX_F64)
        hipLaunchKernelGGL(absmax_rows_kernel<double>, dim3((unsigned)gx, (unsigned)(d + 1)), dim3(256), 0,
                           stream, (const double*)X_t, (const double*)w, absmax, n, d, vec_ok);
    else
        hipLaunchKernelGGL(absmax_rows_kernel<float>, dim3((unsigned)gx, (unsigned)(d + 1)), dim3(256), 0,
                           stream, (const float*)X_t, (const float*)w, absmax, n, d, vec_ok);
    hipLaunchKernelGGL(fixed_point_exponents_kernel, dim3((unsigned)kmx_cdiv(d + 1, 128)), dim3(128), 0,
                       stream, absmax, q_exp, n, d);
    const size_t words = (size_t)(d + 1) * L.k_for_gsum * 2;
    hipLaunchKernelGGL(absmax_zero_kernel, dim3(1), dim3(1024), 0, stream,
                       reinterpret_cast<unsigned int*>(ws + L.off_gsum), (int)words);
    KMX_LAUNCH_CHECK();
    // the screened step compares score gaps with a bound proportional to ||x_i||
    if (L.screen || L.screen64)
        return kmx_sample_norms(X_t, reinterpret_cast<float*>(ws + L.off_bucket + 256), n, d, dtype, stream);
    return KMX_OK;
}

int32_t kmx_lloyd_iter_mfma_f32(const LloydLayout& L, const void* X_t, const void* w,
                                const void* centroids_t, void* new_centroids_t,
                                const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                                uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                                hipStream_t stream, hipEvent_t* events) {
    if (L.acc_mode != KMX_ACC_LDS) return KMX_ERR_UNSUPPORTED;
    LloydTail<float> tail;
    tail.sums_t = (float*)new_centroids_t;
    tail.sizes = (float*)sizes;
    tail.empty_clusters = empty_clusters;
    tail.old_centroids_t = (const float*)centroids_t;
    tail.cpack = reinterpret_cast<float*>(ws + L.off_cpack);
    tail.half_norms = reinterpret_cast<float*>(ws + L.off_half);
    tail.status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    tail.d = d;
    tail.k = k;
    tail.dpad = L.dpad;
    const int* q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
    unsigned long long* gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
    if (events) (void)hipEventRecord(events[0], stream);
    if (L.screen) {
        // labels screened on the fp16 matrix cores (lloyd_mfma_screen.hip)
        uint32_t* uncertain = reinterpret_cast<uint32_t*>(ws + L.off_bucket);
        tail.clear_word = uncertain;
        // Sums corrected instead of rebuilt once an iteration changes at most one label in 3
        // (a sample that moves costs two sets of LDS atomics, one that is rebuilt one).  Up to one
        // change in 24 the step collects the moving samples and fetches them after its last
        // tile; above that the fetch (a 64-byte sector per value) would cost more than a second
        // read of the rows by the tiles.  Measured at 5e6 x 14: a step that rebuilds takes
        // 130 us, one that corrects from the list 91 us plus about 11 us per percent of labels
        // that change.
        tail.n_samples = n;
        tail.delta_divisor = 3;
        tail.list_divisor = 24;
        const int32_t rc = kmx_lloyd_step_mfma_screen(
            X_t, w, centroids_t, labels_prev, labels, tail.status,
            reinterpret_cast<const unsigned int*>(ws + L.off_scales), q_exp, gsum, uncertain,
            reinterpret_cast<const float*>(ws + L.off_bucket + 256), n, d, k, L.wgs_per_cu, stream,
            KMX_SCR_FUSE_TAIL ? &tail : nullptr);
        if (rc != KMX_OK) return rc;
        if (events) {
            (void)hipEventRecord(events[1], stream);
            (void)hipEventRecord(events[2], stream);
        }
        if (KMX_SCR_FUSE_TAIL) {
            // (the step's last workgroup has finished the iteration)
            if (events) (void)hipEventRecord(events[3], stream);
            return KMX_OK;
        }
    } else {
        const int32_t rc = launch_mfma<true>(L, X_t, w, centroids_t, labels_prev, labels,
                                             tail.status, q_exp, gsum, n, d, k, stream);
        if (rc != KMX_OK) return rc;
        if (events) {
            (void)hipEventRecord(events[1], stream);
            (void)hipEventRecord(events[2], stream);
        }
    }
    hipLaunchKernelGGL((lloyd_small_finalize_kernel<float, true>), dim3(1), dim3(256),
                       (size_t)(d + 1) * k * sizeof(float), stream, gsum, q_exp, tail);
    KMX_LAUNCH_CHECK();
    if (events) (void)hipEventRecord(events[3], stream);
    return KMX_OK;
}

// fp64 inputs: the screened fused step (lloyd_mfma_screen.hip), whose last workgroup finishes
// the iteration.
int32_t kmx_lloyd_iter_mfma_screen_f64(const LloydLayout& L, const void* X_t, const void* w,
                                       const void* centroids_t, void* new_centroids_t,
                                       const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                                       uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                                       hipStream_t stream, hipEvent_t* events) {
    if (!L.screen64) return KMX_ERR_UNSUPPORTED;
    LloydTail<double> tail;
    tail.sums_t = (double*)new_centroids_t;
    tail.sizes = (double*)sizes;
    tail.empty_clusters = empty_clusters;
    tail.old_centroids_t = (const double*)centroids_t;
    tail.cpack = reinterpret_cast<double*>(ws + L.off_cpack);
    tail.half_norms = reinterpret_cast<double*>(ws + L.off_half);
    tail.status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    tail.d = d;
    tail.k = k;
    tail.dpad = L.dpad;
    const int* q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
    unsigned long long* gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
    uint32_t* uncertain = reinterpret_cast<uint32_t*>(ws + L.off_bucket);
    tail.clear_word = uncertain;
    tail.n_samples = n;
    tail.delta_divisor = 3;  // (as for fp32 inputs)
    tail.list_divisor = 24;
    if (events) (void)hipEventRecord(events[0], stream);
    const int32_t rc = kmx_lloyd_step_mfma_screen_f64(
        X_t, w, centroids_t, labels_prev, labels, tail.status,
        reinterpret_cast<const unsigned int*>(ws + L.off_scales), q_exp, gsum, uncertain,
        reinterpret_cast<const float*>(ws + L.off_bucket + 256), n, d, k, L.wgs_per_cu, stream, &tail);
    if (rc != KMX_OK) return rc;
    if (events)
        for (int i = 1; i < 4; ++i) (void)hipEventRecord(events[i], stream);
    return KMX_OK;
}

int32_t kmx_assign_labels_mfma_f32(const LloydLayout& L, const void* X_t, const void* centroids_t,
                                   uint32_t* labels, char* ws, int64_t n, int d, int k,
                                   hipStream_t stream) {
    (void)ws;
    return launch_mfma<false>(L, X_t, nullptr, centroids_t, nullptr, labels, nullptr, nullptr,
                              nullptr, n, d, k, stream);
}
