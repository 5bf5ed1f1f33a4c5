// fp32 fused Lloyd step whose label assignment is SCREENED on the fp16 matrix cores of gfx950
// (v_mfma_f32_32x32x16_f16, 16x the rate of the fp32 MFMA) and CERTIFIED per sample.
//
// X and the centroids are scaled by one power of two, 2^-a, that brings max|x| into
// [2^14, 2^15) (exact, and it leaves the arg-max unchanged).  Every scaled value is split into
// two fp16 numbers, v = hi + lo + rest, by two round-to-nearest conversions (the subtraction
// v - hi is exact): |rest| <= 2^-22 |v|, or at most 2^-14 in absolute terms should the
// hardware flush fp16 subnormals.  The score of sample x against centroid c,
// <x, c> - 0.5||c||^2, is approximated by three fp16 products accumulated in fp32,
// hi*hi + lo*hi + hi*lo, started at -0.5||c||^2.  What is left out is
//   x_lo c_lo + (x - x_rest) c_rest + x_rest c  <=  3.01 * 2^-22 * sum_f |x_f c_f| + (absolute part),
// and the fp32 accumulation of the 48 exact products adds at most 51 roundings of one ulp of a
// partial sum each (6.1e-6 relative to 0.5||c||^2 + sum_f |x_f c_f|).  With Cauchy-Schwarz the
// error of every score of sample x is bounded by
//   E(x) = 6.93e-6 ||x|| C + 6.2e-6 H + 6.2e-5 sqrt(d) (||x|| + C),  C = max ||c||, H = max 0.5||c||^2
// (scaled units).  If the best approximate score beats the second best by more than 2 E(x),
// the arg-max of the approximate scores IS the arg-max of the exact real-valued scores: the
// label is certain.  Otherwise (about 2 samples in 1000 on blob data) the sample is put on a
// list and left out of the sums, and `lloyd_recheck_kernel` evaluates it in plain fp32
// (feature-sequential fused multiply-adds, lowest index wins a tie) and adds it to the sums.
// Labels therefore meet the same bar as an all-fp32 evaluation (they can differ from it only
// where fp32's own rounding decides), and the sums are taken from the fp32 inputs in 64-bit
// fixed point exactly as in lloyd_mfma.hip.  Non-finite scores make a sample uncertain.
//
// Work decomposition: as in lloyd_mfma.hip with two sample columns per lane.  Lane (j, h) of a
// wave owns features 16 s + 2 i + h (i < 8) of samples 2 j, 2 j + 1 of the wave's 64-sample
// tile: slot i of half-wave h is K index 8 h + i of K step s for both MFMA operands.
#include "lloyd_layout.h"
#include "lloyd_tail.h"

#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef double v8d __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr double FIX_MAGIC = 6755399441055744.0;  // 1.5 * 2^52
constexpr long long FIX_MAGIC_BITS = 0x4338000000000000ll;
__device__ __forceinline__ unsigned long long to_fixed(double scaled_plus_magic) {
    return (unsigned long long)(__double_as_longlong(scaled_plus_magic) - FIX_MAGIC_BITS);
}

// Error bound of one approximate score, in scaled units:
//   SCR_ERR_X ||x|| C + SCR_ERR_H H + SCR_ERR_ABS sqrt(d) (||x|| + C)
constexpr float SCR_ERR_X = 6.93e-6f;
constexpr float SCR_ERR_H = 6.2e-6f;
constexpr float SCR_ERR_ABS = 6.2e-5f;
constexpr int SCR_QUEUE = 1024;  // uncertain samples a workgroup buffers in LDS
constexpr int SCR_GROUP = 8;  // accumulator registers per arg-max group

// Waves per workgroup (one workgroup per compute unit, or two of four waves).
#ifndef KMX_SCR_WAVES
#define KMX_SCR_WAVES 8
#endif
constexpr int scr_waves(int nk) { return nk == 1 ? KMX_SCR_WAVES : 4; }

struct ScreenLds {
    size_t off_afh, off_afl, off_hneg, off_queue, total;
};
__host__ __device__ inline ScreenLds screen_lds(int d, int k, int nk, bool update) {
    ScreenLds s;
    const size_t n_cb = (size_t)(k + 31) / 32;
    const size_t acc = update ? (((size_t)(d + 1) * k * 8 + 15) & ~(size_t)15) : 0;
    s.off_afh = acc;
    s.off_afl = s.off_afh + n_cb * nk * 64 * 16;
    s.off_hneg = s.off_afl + n_cb * nk * 64 * 16;
    s.off_queue = s.off_hneg + n_cb * 32 * 4;
    s.total = s.off_queue + (size_t)SCR_QUEUE * 4;
    return s;
}

// 1.5 * 2^(52 - q): adding it to |v| < 2^(51 - q) leaves round-to-nearest(v * 2^q) in the low
// mantissa bits, so the product x * w needs no separate scaling by 2^q.  The low word is zero.
__device__ __forceinline__ double fix_magic(int q) {
    return __hiloint2double((int)(0x43380000u - ((unsigned int)q << 20)), 0);
}
__device__ __forceinline__ unsigned long long to_fixed_q(double v_plus_magic, double magic) {
    // only the high words differ (asm: the optimiser would rebuild a 64-bit subtraction)
    unsigned int hi;
    asm("v_sub_u32 %0, %1, %2" : "=v"(hi) : "v"(__double2hiint(v_plus_magic)), "v"(__double2hiint(magic)));
    return ((unsigned long long)hi << 32) | (unsigned int)__double2loint(v_plus_magic);
}

template <int NK, bool UPDATE>
__global__ __launch_bounds__(64 * scr_waves(NK)) void lloyd_screen_kernel(
    const float* __restrict__ X_t, const float* __restrict__ sample_weight,
    const float* __restrict__ centroids_t, const uint32_t* __restrict__ labels_prev,
    uint32_t* __restrict__ labels, kmx_lloyd_status* __restrict__ status,
    const unsigned int* __restrict__ absmax, const int* __restrict__ q_exp,
    unsigned long long* __restrict__ gsum, uint32_t* __restrict__ recheck_list,
    uint32_t* __restrict__ recheck_count, int64_t n, int d, int k, int vec_ok) {
    if (UPDATE && status->state != KMX_RUNNING) return;

    constexpr int WAVES = scr_waves(NK), THREADS = 64 * WAVES;
    constexpr int MC = 2, TILE = 64;
    constexpr int G = SCR_GROUP, NG = 16 / SCR_GROUP;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int n_cb = (k + 31) >> 5;
    const int items = (d + 1) * k;
    const ScreenLds lay = screen_lds(d, k, NK, UPDATE);
    unsigned long long* acc = reinterpret_cast<unsigned long long*>(smem_raw);  // [(d + 1) * k]
    v8h* afh = reinterpret_cast<v8h*>(smem_raw + lay.off_afh);                  // [n_cb][NK][64]
    v8h* afl = reinterpret_cast<v8h*>(smem_raw + lay.off_afl);
    float* hneg = reinterpret_cast<float*>(smem_raw + lay.off_hneg);            // [n_cb][2][16]
    uint32_t* queue = reinterpret_cast<uint32_t*>(smem_raw + lay.off_queue);    // [SCR_QUEUE]
    __shared__ unsigned int changed_block;
    __shared__ unsigned int hmax_bits;
    __shared__ unsigned int queue_count;
    __shared__ unsigned int queue_base;

    if (threadIdx.x == 0) {
        changed_block = 0;
        hmax_bits = 0;
        queue_count = 0;
    }
    // a batch that does not fit the queue goes to the global list and leaves a hole here
    for (int q = threadIdx.x; q < SCR_QUEUE; q += THREADS) queue[q] = 0xffffffffu;
    // 2^-a with max|x| * 2^-a in [2^14, 2^15) (1 for all-zero or non-finite data)
    float xmax = 0.0f;
    for (int f = 0; f < d; ++f) xmax = fmaxf(xmax, __uint_as_float(absmax[f]));
    const float xs = (xmax > 0.0f && xmax < kmx_inf<float>()) ? ldexpf(1.0f, 14 - ilogbf(xmax)) : 1.0f;
    __syncthreads();
    // A operand: hi and lo parts of 32 centroids x 16 features per block and K step
    for (int idx = threadIdx.x; idx < n_cb * NK * 64; idx += THREADS) {
        const int l = idx & 63;
        const int s = (idx >> 6) % NK;
        const int cb = (idx >> 6) / NK;
        const int c = 32 * cb + (l & 31);
        v8h hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = 16 * s + 2 * i + (l >> 5);
            const float v = (c < k && f < d) ? centroids_t[(size_t)f * k + c] * xs : 0.0f;
            const _Float16 hb = (_Float16)v;
            hi[i] = hb;
            lo[i] = (_Float16)(v - (float)hb);
        }
        afh[idx] = hi;
        afl[idx] = lo;
    }
    for (int idx = threadIdx.x; idx < n_cb * 32; idx += THREADS) {
        const int cb = idx >> 5, hh = (idx >> 4) & 1, r = idx & 15;
        const int c = 32 * cb + 8 * (r >> 2) + 4 * hh + (r & 3);
        float v = -kmx_inf<float>();
        if (c < k) {
            float sq = 0.0f;
            for (int f = 0; f < d; ++f) {
                const float cv = centroids_t[(size_t)f * k + c] * xs;
                sq += cv * cv;
            }
            v = -(sq / 2.0f);
            // non-negative floats order like their bits; a NaN norm ends up as the maximum
            // and makes every sample uncertain
            atomicMax(&hmax_bits, __float_as_uint(sq / 2.0f));
        }
        hneg[idx] = v;
    }
    if (UPDATE)
        for (int jx = threadIdx.x; jx < items; jx += THREADS) acc[jx] = 0ull;
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int64_t n_wtiles = (n + TILE - 1) / TILE;
    unsigned int changed = 0;

    // uncertain when best - second <= thr_x * ||x|| + thr_0: twice the error bound, with a
    // margin for the rounding of the bound itself and of the hardware square root
    const float hmax = __uint_as_float(hmax_bits);
    const float cmax = sqrtf(2.0f * hmax), abs_term = SCR_ERR_ABS * sqrtf((float)d);
    const float thr_x = 2.01f * (SCR_ERR_X * cmax + abs_term);
    const float thr_0 = 2.01f * (SCR_ERR_H * hmax + abs_term * cmax);
    // +inf the optimiser cannot see through (it would turn the median below into a maximum
    // with two canonicalising instructions in front)
    float pos_inf = kmx_inf<float>();
    asm volatile("" : "+s"(pos_inf));
    const float neg_inf = -kmx_inf<float>();

    // The lane's features: pair p = 8 s + i, feature 2 p + h.  xsr: 2^-a, or 0 for a feature
    // that does not exist (its loads read row d - 1); magic: see fix_magic.
    float xsr[NK][8];
    double magic[NK][8];
    double magic_w = 0.0;
#pragma unroll
    for (int s = 0; s < NK; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = 16 * s + 2 * i + h;
            xsr[s][i] = f < d ? xs : 0.0f;
            magic[s][i] = 0.0;
            if (UPDATE) magic[s][i] = fix_magic(f < d ? q_exp[f] : 0);
        }
    if (UPDATE) magic_w = fix_magic(q_exp[d]);

    // One tile of NC sample columns per lane (NC = 2: samples i0, i0 + 1; NC = 1: sample i0).
    // x holds the lane's rows at its samples (row d - 1 where the feature does not exist).
    auto process = [&](auto nc_tag, auto full_tag,
                       const float(&x)[NK][8][decltype(nc_tag)::value],
                       const float(&wv)[decltype(nc_tag)::value],
                       const uint32_t(&pl)[decltype(nc_tag)::value], const int64_t i0) {
        constexpr int NC = decltype(nc_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;

        // scaled fp16 split of the B operand and ||x||^2
        v8h xh[NK][NC], xl[NK][NC];
        float nrm[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            float ss = 0.0f;
#pragma unroll
            for (int s = 0; s < NK; ++s)
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    const v2f p = {x[s][i][t] * xsr[s][i], x[s][i + 1][t] * xsr[s][i + 1]};
                    const v2h hh = __builtin_convertvector(p, v2h);
                    const v2f r = p - __builtin_convertvector(hh, v2f);
                    const v2h ll = __builtin_convertvector(r, v2h);
                    xh[s][t][i] = hh[0];
                    xh[s][t][i + 1] = hh[1];
                    xl[s][t][i] = ll[0];
                    xl[s][t][i + 1] = ll[1];
                    ss = fmaf(p[0], p[0], ss);
                    ss = fmaf(p[1], p[1], ss);
                }
            nrm[t] = ss + __shfl_xor(ss, 32, 64);
        }

        // Running arg-max by groups of G accumulator registers, plus the second largest of
        // the group maxima (the median of best, second and the new maximum).
        float best[NC], second[NC];
        unsigned int code[NC];
        // the winning group's registers, as pairs; whatever the registers hold until the first
        // group with a score above -inf overwrites them (no instruction spent on a reset)
        double svd[NC][G / 2];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            best[t] = neg_inf;
            second[t] = neg_inf;
            code[t] = 0;
#pragma unroll
            for (int r = 0; r < G / 2; ++r) asm volatile("" : "=v"(svd[t][r]));
        }

        // approximate scores of centroid block cb for the NC columns
        auto scores = [&](const int cb, v16f(&a)[NC]) __attribute__((always_inline)) {
            const float4* hp = reinterpret_cast<const float4*>(hneg + cb * 32 + h * 16);
            v16f hv;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 v4 = hp[q];
                hv[4 * q] = v4.x;
                hv[4 * q + 1] = v4.y;
                hv[4 * q + 2] = v4.z;
                hv[4 * q + 3] = v4.w;
            }
#pragma unroll
            for (int s = 0; s < NK; ++s) {
                const v8h ah = afh[(cb * NK + s) * 64 + lane];
                const v8h al = afl[(cb * NK + s) * 64 + lane];
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    a[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xh[s][t], s == 0 ? hv : a[t], 0, 0, 0);
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    a[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xl[s][t], a[t], 0, 0, 0);
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    a[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, xh[s][t], a[t], 0, 0, 0);
            }
        };
        auto argmax_block = [&](const int cb, const v16f(&a)[NC]) __attribute__((always_inline)) {
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const unsigned int cd = (unsigned int)(cb * NG + g);  // wave-uniform
#pragma unroll
                for (int t = 0; t < NC; ++t) {
                    // The first read of the matrix-core result is an instruction the compiler
                    // knows (the median of a, b and +inf is max(a, b)): it inserts the wait
                    // states an MFMA result needs before a vector-ALU read, which it does not
                    // do for operands of inline assembly.
                    float m = __builtin_amdgcn_fmed3f(a[t][g * G], a[t][g * G + 1], pos_inf);
#pragma unroll
                    for (int r = 2; r + 1 < G; r += 2)
                        asm("v_max3_f32 %0, %1, %2, %3"
                            : "=v"(m)
                            : "v"(m), "v"(a[t][g * G + r]), "v"(a[t][g * G + r + 1]));
                    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(second[t]) : "v"(best[t]), "v"(second[t]), "v"(m));
                    // strict: the earlier group keeps a tie
                    if (m > best[t]) {
                        best[t] = m;
                        code[t] = cd;
                        const v8d ad = __builtin_bit_cast(v8d, a[t]);
#pragma unroll
                        for (int r = 0; r < G / 2; ++r)
                            asm volatile("v_mov_b64 %0, %1" : "+v"(svd[t][r]) : "v"(ad[g * (G / 2) + r]));
                    }
                }
            }
        };
        for (int cb = 0; cb < n_cb; ++cb) {
            v16f a[NC];
            scores(cb, a);
            argmax_block(cb, a);
        }

        // position inside the winning group, second largest inside it, then both half-waves
        uint32_t lab[NC];
        bool unsure[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            float sv[G];
#pragma unroll
            for (int r = 0; r < G / 2; ++r) {
                const float2 pr = __builtin_bit_cast(float2, svd[t][r]);
                sv[2 * r] = pr.x;
                sv[2 * r + 1] = pr.y;
            }
            // registers equal to the best: the lowest is the label's; a second one makes the
            // second best equal to the best
            unsigned int pos = G - 1, pos_hi = 0;
            float rest[G];
#pragma unroll
            for (int r = G - 1; r >= 0; --r) {
                const bool eq = sv[r] == best[t];
                pos = eq ? (unsigned int)r : pos;
                pos_hi = eq ? (unsigned int)(G - 1 - r) : pos_hi;  // ends as the highest match, mirrored
                rest[r] = eq ? neg_inf : sv[r];
            }
            float sec = second[t];
#pragma unroll
            for (int r = 0; r + 1 < G; r += 2)
                asm("v_max3_f32 %0, %1, %2, %3" : "=v"(sec) : "v"(sec), "v"(rest[r]), "v"(rest[r + 1]));
            sec = (pos + pos_hi != (unsigned int)(G - 1)) ? best[t] : sec;
            const unsigned int reg = (code[t] % NG) * G + pos;
            const unsigned int blk = code[t] / NG;
            int c = (int)(32 * blk + 8 * (reg >> 2) + 4 * h + (reg & 3));
            const float ov = __shfl_xor(best[t], 32, 64);
            const float o2 = __shfl_xor(sec, 32, 64);
            const int oc = __shfl_xor(c, 32, 64);
            // second best over both halves: the loser of the two bests or a half's own second
            float s2 = sec > o2 ? sec : o2;
            const float lo_best = ov < best[t] ? ov : best[t];
            s2 = lo_best > s2 ? lo_best : s2;
            float b = best[t];
            if (ov > b || (ov == b && oc < c)) {
                c = oc;
                b = ov;
            }
            lab[t] = (uint32_t)c;
            // written so that a NaN anywhere makes the sample uncertain
            const float thr = fmaf(thr_x, __builtin_amdgcn_sqrtf(nrm[t]), thr_0);
            unsure[t] = !(b - s2 > thr) && (FULL || i0 + t < n);
        }

        if (h == 0) {
            if constexpr (FULL && NC == 2) {
                *reinterpret_cast<uint2*>(labels + i0) = make_uint2(lab[0], lab[1]);
            } else {
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    if (FULL || i0 + t < n) labels[i0 + t] = lab[t];
            }
        }

        // uncertain samples go on the list (lower half-wave only: both halves hold the same flags)
        unsigned long long um[NC];
        int n_unsure = 0;
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            um[t] = __ballot(h == 0 && unsure[t]);
            n_unsure += __popcll(um[t]);
        }
        if (n_unsure) {  // wave-uniform
            // into the workgroup's queue, or straight to the global list when that is full
            unsigned int base = 0;
            if (lane == 0) base = atomicAdd(&queue_count, (unsigned int)n_unsure);
            base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
            uint32_t* dst = queue;
            if (base + (unsigned int)n_unsure > (unsigned int)SCR_QUEUE) {
                if (lane == 0) base = atomicAdd(recheck_count, (unsigned int)n_unsure);
                base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
                dst = recheck_list;
            }
            const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                if (h == 0 && unsure[t]) dst[base + __popcll(um[t] & below)] = (uint32_t)(i0 + t);
                base += __popcll(um[t]);
            }
        }

        if (UPDATE) {
            if (h == 0) {
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    changed += ((FULL || i0 + t < n) && !unsure[t] && pl[t] != lab[t]) ? 1u : 0u;
            }
            // uncertain samples and samples past the end add zero
            double wd[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) wd[t] = unsure[t] ? 0.0 : (double)wv[t];
#pragma unroll
            for (int s = 0; s < NK; ++s)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int p0 = 16 * s + 2 * i;  // the pair's even feature
                    if (p0 < d) {                   // wave-uniform
                        // odd d, last pair: the upper half-wave adds zero to row d - 1
                        const bool odd_tail = p0 + 1 == d;
                        unsigned long long* rowacc = acc + (odd_tail ? p0 : p0 + h) * k;
#pragma unroll
                        for (int t = 0; t < NC; ++t) {
                            const double xd = (double)((odd_tail && h) ? 0.0f : x[s][i][t]);
                            // x * w is exact in fp64; one rounding, to a multiple of 2^-q
                            const double v = fma(xd, wd[t], magic[s][i]);
                            atomicAdd(rowacc + lab[t], to_fixed_q(v, magic[s][i]));
                        }
                    }
                }
            if (h == 0) {
                unsigned long long* szacc = acc + d * k;
#pragma unroll
                for (int t = 0; t < NC; ++t)
                    atomicAdd(szacc + lab[t], to_fixed_q(wd[t] + magic_w, magic_w));
            }
        }
    };
    using Cols2 = std::integral_constant<int, MC>;
    using Cols1 = std::integral_constant<int, 1>;

    const int64_t wt_step = (int64_t)gridDim.x * WAVES;
    const int64_t wt_first = (int64_t)blockIdx.x * WAVES + wave;
    const int64_t n_fast = vec_ok ? n / TILE : 0;
    // a last round of full tiles that is at most three quarters full is cut into
    // single-column tiles of 32 samples, spread over all the waves
    const int64_t n_rounds = n_fast / wt_step;
    const int64_t n_left = n_fast - n_rounds * wt_step;
    const bool halves = n_left > 0 && 4 * n_left <= 3 * wt_step;
    const int64_t n_main = halves ? n_rounds * wt_step : n_fast;

    // Rows of the lane: feature 2 p + h for the pairs p = 8 s + i.  Every load is a uniform
    // row address plus a 32-bit byte offset of the lane (n < 2^29), and unconditional, so
    // that the compiler counts the loads and waits for the older tile only: a pair that is
    // not entirely below d reads row d - 1 in both half-waves.
    const char* const xbytes = reinterpret_cast<const char*>(X_t);
    uint32_t lane_off[NK][8];
#pragma unroll
    for (int s = 0; s < NK; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i)
            lane_off[s][i] = (uint32_t)(MC * j) * 4u + ((16 * s + 2 * i + 1 < d) ? (uint32_t)h * (uint32_t)n * 4u : 0u);
    auto load_rows = [&](const int64_t wt, float(&dst)[NK][8][MC]) {
        const uint32_t tile_off = (uint32_t)wt * (uint32_t)(TILE * 4);
#pragma unroll
        for (int s = 0; s < NK; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int p0 = 16 * s + 2 * i;
                const char* row = xbytes + (size_t)(p0 + 1 < d ? p0 : d - 1) * (size_t)n * 4u;
                const float2 q = *reinterpret_cast<const float2*>(row + (tile_off + lane_off[s][i]));
                dst[s][i][0] = q.x;
                dst[s][i][1] = q.y;
            }
    };

    if (wt_first < n_main) {
        float xn[NK][8][MC];
        load_rows(wt_first, xn);
        for (int64_t wt = wt_first; wt < n_main; wt += wt_step) {
            const int64_t i0 = wt * TILE + MC * j;
            float x[NK][8][MC];
#pragma unroll
            for (int s = 0; s < NK; ++s)
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int t = 0; t < MC; ++t) x[s][i][t] = xn[s][i][t];
            // past the last tile the same rows are read again (and not used)
            load_rows(wt + wt_step < n_main ? wt + wt_step : wt, xn);
            float wv[MC] = {0.f, 0.f};
            uint32_t pl[MC] = {0u, 0u};
            if (UPDATE) {
                const float2 w2 = *reinterpret_cast<const float2*>(sample_weight + i0);
                wv[0] = w2.x;
                wv[1] = w2.y;
                const uint2 p2 = *reinterpret_cast<const uint2*>(labels_prev + i0);
                pl[0] = p2.x;
                pl[1] = p2.y;
            }
            process(Cols2{}, std::true_type{}, x, wv, pl, i0);
        }
    }
    // scalar loads of the lane's rows (row d - 1 where the feature does not exist)
    auto load_scalar = [&](auto nc_tag, const int64_t i0, float(&dst)[NK][8][decltype(nc_tag)::value]) {
        constexpr int NC = decltype(nc_tag)::value;
#pragma unroll
        for (int s = 0; s < NK; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int f = 16 * s + 2 * i + h;
                const float* row = X_t + (size_t)(f < d ? f : d - 1) * n;
#pragma unroll
                for (int t = 0; t < NC; ++t) dst[s][i][t] = i0 + t < n ? row[i0 + t] : 0.0f;
            }
    };
    if (halves) {
        // single-column tile q of the left-over tiles: samples [n_main * TILE + 32 q, + 32)
        for (int64_t q = wt_first; q < MC * n_left; q += wt_step) {
            const int64_t i0 = n_main * TILE + 32 * q + j;
            float x[NK][8][1];
            load_scalar(Cols1{}, i0, x);
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
        float x[NK][8][MC];
        load_scalar(Cols2{}, i0, x);
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
        process(Cols2{}, std::false_type{}, x, wv, pl, i0);
    }

    if (UPDATE && changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    // the queue (holes included: the recheck skips them) moves to the global list
    const unsigned int q_n = queue_count < (unsigned int)SCR_QUEUE ? queue_count : (unsigned int)SCR_QUEUE;
    if (threadIdx.x == 0 && q_n) queue_base = atomicAdd(recheck_count, q_n);
    __syncthreads();
    for (unsigned int q = threadIdx.x; q < q_n; q += THREADS) recheck_list[queue_base + q] = queue[q];
    if (UPDATE) {
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
        for (int jx = threadIdx.x; jx < items; jx += THREADS) {
            const unsigned long long v = acc[jx];
            if (v) atomicAdd(gsum + jx, v);
        }
    }
}

// ---------------------------------------------------------------------------- recheck

constexpr int RECHECK_THREADS = 256;
constexpr int RECHECK_PARTS = 4;  // lanes per sample, each takes every fourth centroid
constexpr int RECHECK_CHUNK = RECHECK_THREADS / RECHECK_PARTS;  // samples per block and pass
constexpr int RECHECK_BLOCKS = 1024;

__host__ __device__ inline size_t recheck_lds_bytes(int d, int k, int dpad, bool update) {
    size_t b = update ? (((size_t)(d + 1) * k * 8 + 15) & ~(size_t)15) : 0;
    b += (size_t)k * dpad * 4 + (size_t)k * 4 + (size_t)(d + 1) * 4;
    return b;
}

// The listed samples in plain fp32: score = -0.5||c||^2 + sum_f x_f c_f by fused multiply-adds
// in feature order, strict '>' in increasing centroid order.  Four neighbouring lanes share a
// sample (centroids p, p + 4, ... each, combined with the lowest index winning a tie); block b
// takes the chunks b, b + gridDim.x, ... of the list, and blocks without a chunk leave at once.
// Entries 0xffffffff are holes.
template <int NK, bool UPDATE>
__global__ __launch_bounds__(RECHECK_THREADS) void lloyd_recheck_kernel(
    const float* __restrict__ X_t, const float* __restrict__ sample_weight,
    const float* __restrict__ cpack, const float* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    const uint32_t* __restrict__ recheck_list, const uint32_t* __restrict__ recheck_count,
    kmx_lloyd_status* __restrict__ status, const int* __restrict__ q_exp,
    unsigned long long* __restrict__ gsum, int64_t n, int d, int k, int dpad) {
    if (UPDATE && status->state != KMX_RUNNING) return;
    const uint32_t cnt = *recheck_count;
    if ((uint64_t)blockIdx.x * RECHECK_CHUNK >= cnt) return;

    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int items = (d + 1) * k;
    unsigned long long* acc = reinterpret_cast<unsigned long long*>(smem_raw);
    float* cp = reinterpret_cast<float*>(smem_raw + (UPDATE ? (((size_t)items * 8 + 15) & ~(size_t)15) : 0));
    float* hn = cp + (size_t)k * dpad;
    float* qscale = hn + k;
    __shared__ unsigned int changed_block;
    for (int idx = threadIdx.x; idx < k * dpad; idx += RECHECK_THREADS) cp[idx] = cpack[idx];
    for (int c = threadIdx.x; c < k; c += RECHECK_THREADS) hn[c] = half_norms[c];
    if (UPDATE) {
        for (int jx = threadIdx.x; jx < items; jx += RECHECK_THREADS) acc[jx] = 0ull;
        for (int f = threadIdx.x; f <= d; f += RECHECK_THREADS) qscale[f] = ldexpf(1.0f, q_exp[f]);
        if (threadIdx.x == 0) changed_block = 0;
    }
    __syncthreads();

    const int part = threadIdx.x & (RECHECK_PARTS - 1), slot = threadIdx.x / RECHECK_PARTS;
    unsigned int changed = 0;
    for (uint64_t base = (uint64_t)blockIdx.x * RECHECK_CHUNK; base < cnt;
         base += (uint64_t)gridDim.x * RECHECK_CHUNK) {
        const uint64_t e = base + slot;
        const uint32_t entry = e < cnt ? recheck_list[e] : 0xffffffffu;
        const bool active = entry != 0xffffffffu;
        const int64_t i = active ? (int64_t)entry : 0;
        float x[16 * NK];
#pragma unroll
        for (int f = 0; f < 16 * NK; ++f) x[f] = f < d ? X_t[(size_t)f * n + i] : 0.0f;
        float best = -kmx_inf<float>();
        int bl = 0x7fffffff;
        for (int c = part; c < k; c += RECHECK_PARTS) {
            const float4* __restrict__ row = reinterpret_cast<const float4*>(cp + (size_t)c * dpad);
            float s = -hn[c];
#pragma unroll
            for (int f4 = 0; f4 < 4 * NK; ++f4)
                if (4 * f4 < dpad) {  // wave-uniform; the padding of the packed rows is zero
                    const float4 q = row[f4];
                    s = fmaf(x[4 * f4], q.x, s);
                    s = fmaf(x[4 * f4 + 1], q.y, s);
                    s = fmaf(x[4 * f4 + 2], q.z, s);
                    s = fmaf(x[4 * f4 + 3], q.w, s);
                }
            if (s > best) {
                best = s;
                bl = c;
            }
        }
#pragma unroll
        for (int off = 1; off < RECHECK_PARTS; off <<= 1) {
            const float ov = __shfl_xor(best, off, 64);
            const int oc = __shfl_xor(bl, off, 64);
            if (ov > best || (ov == best && oc < bl)) {
                best = ov;
                bl = oc;
            }
        }
        if (bl == 0x7fffffff) bl = 0;  // every score NaN: the reference's running arg-min keeps 0
        if (active) {
            if (part == 0) {
                labels[i] = (uint32_t)bl;
                if (UPDATE) changed += labels_prev[i] != (uint32_t)bl ? 1u : 0u;
            }
            if (UPDATE) {
                const double wd = (double)sample_weight[i];
#pragma unroll
                for (int f = 0; f < 16 * NK; ++f)
                    if (f < d && (f & (RECHECK_PARTS - 1)) == part) {
                        const double v = fma((double)x[f], wd * (double)qscale[f], FIX_MAGIC);
                        atomicAdd(acc + f * k + bl, to_fixed(v));
                    }
                if (part == RECHECK_PARTS - 1)
                    atomicAdd(acc + d * k + bl, to_fixed(fma(wd, (double)qscale[d], FIX_MAGIC)));
            }
        }
    }
    if (UPDATE) {
        if (changed) atomicAdd(&changed_block, changed);
        __syncthreads();
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
        for (int jx = threadIdx.x; jx < items; jx += RECHECK_THREADS) {
            const unsigned long long v = acc[jx];
            if (v) atomicAdd(gsum + jx, v);
        }
    }
}

}  // namespace

// Shapes the screened step covers: d <= 32, the operands of both kernels within 64 KB of LDS,
// byte offsets inside two rows of X_t within 32 bits.  KMX_LLOYD_ASSIGN = f32 switches it off (all-fp32 scores).
bool kmx_mfma_screen_supported(int64_t n, int d, int k) {
    if (d < 1 || d > 32 || k < 16 || n >= ((int64_t)1 << 29)) return false;
    const char* v = std::getenv("KMX_LLOYD_ASSIGN");
    if (v != nullptr && std::strcmp(v, "f32") == 0) return false;
    const int nk = (d + 15) / 16, dpad = (d + 3) & ~3;
    return screen_lds(d, k, nk, true).total <= 64 * 1024 &&
           recheck_lds_bytes(d, k, dpad, true) <= 64 * 1024;
}

// Screened fused step + recheck of the uncertain samples.  `recheck` points at the counter
// (one word, zero on entry; the finalisation that follows clears it again) followed, 64 words
// later, by room for n + KMX_SCREEN_LIST_SLACK entries (sample indices and the holes of the
// workgroup queues).  `absmax`: bits of max|X_t row| per feature, as kmx_lloyd_mfma_prepare
// leaves them.
int32_t kmx_lloyd_step_mfma_screen(const void* X_t, const void* w, const void* centroids_t,
                                   const void* cpack, const void* half_norms,
                                   const uint32_t* labels_prev, uint32_t* labels,
                                   kmx_lloyd_status* status, const unsigned int* absmax,
                                   const int* q_exp, unsigned long long* gsum, uint32_t* recheck,
                                   int64_t n, int d, int k, int dpad, hipStream_t stream,
                                   hipEvent_t mid_event) {
    if (!kmx_mfma_screen_supported(n, d, k)) return KMX_ERR_UNSUPPORTED;
    const int nk = (d + 15) / 16;
    const int waves = scr_waves(nk);
    const int64_t n_wtiles = kmx_cdiv(n, 64);
    int64_t grid = kmx_cdiv(n_wtiles, waves);
    const int per_cu = waves >= 8 ? 1 : 2;
    const int cap = (kmx_wgs_per_cu_env() > 0 ? kmx_wgs_per_cu_env() : per_cu) * kmx_num_cus();
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
    auto aligned16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    const int vec_ok = (n % 4 == 0) && aligned16(X_t) && aligned16(labels) && aligned16(w) &&
                       aligned16(labels_prev);
    const size_t lds = screen_lds(d, k, nk, true).total;
    uint32_t* count = recheck;
    uint32_t* list = recheck + 64;
    if (nk == 1)
        hipLaunchKernelGGL((lloyd_screen_kernel<1, true>), dim3((unsigned)grid), dim3(64 * scr_waves(1)),
                           lds, stream, (const float*)X_t, (const float*)w, (const float*)centroids_t,
                           labels_prev, labels, status, absmax, q_exp, gsum, list, count, n, d, k, vec_ok);
    else
        hipLaunchKernelGGL((lloyd_screen_kernel<2, true>), dim3((unsigned)grid), dim3(64 * scr_waves(2)),
                           lds, stream, (const float*)X_t, (const float*)w, (const float*)centroids_t,
                           labels_prev, labels, status, absmax, q_exp, gsum, list, count, n, d, k, vec_ok);
    KMX_LAUNCH_CHECK();
    if (mid_event) (void)hipEventRecord(mid_event, stream);
    const size_t lds2 = recheck_lds_bytes(d, k, dpad, true);
    if (nk == 1)
        hipLaunchKernelGGL((lloyd_recheck_kernel<1, true>), dim3(RECHECK_BLOCKS), dim3(RECHECK_THREADS),
                           lds2, stream, (const float*)X_t, (const float*)w, (const float*)cpack,
                           (const float*)half_norms, labels_prev, labels, list, count, status, q_exp,
                           gsum, n, d, k, dpad);
    else
        hipLaunchKernelGGL((lloyd_recheck_kernel<2, true>), dim3(RECHECK_BLOCKS), dim3(RECHECK_THREADS),
                           lds2, stream, (const float*)X_t, (const float*)w, (const float*)cpack,
                           (const float*)half_norms, labels_prev, labels, list, count, status, q_exp,
                           gsum, n, d, k, dpad);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
