// Fused Lloyd step (fp32 or fp64 inputs) whose label assignment is SCREENED on the fp16 matrix cores of gfx950
// (v_mfma_f32_32x32x16_f16, 16x the rate of the fp32 MFMA) and CERTIFIED per sample.
//
// X and the centroids are scaled by one power of two, 2^-a, that brings max|x| into
// [2^12, 2^13) (exact, and it leaves the arg-max unchanged).  Every scaled value is split into
// two fp16 numbers, v = hi + lo + rest, by two round-to-nearest conversions (the subtraction
// v - hi is exact): |rest| <= 2^-22 |v|, or at most 2^-14 in absolute terms should the
// hardware flush fp16 subnormals.  The score of sample x against centroid c,
// <x, c> - 0.5||c||^2, is approximated by three fp16 products accumulated in fp32,
// hi*hi + lo*hi + hi*lo, started at -0.5||c||^2.  What is left out is
//   x_lo c_lo + (x - x_rest) c_rest + x_rest c  <=  3.01 * 2^-22 * sum_f |x_f c_f| + (absolute part),
// and the fp32 accumulation of the 48 exact products adds at most 51 roundings of one ulp of a
// partial sum each (6.1e-6 relative to 0.5||c||^2 + sum_f |x_f c_f|).  With Cauchy-Schwarz the
// error of every score of sample x is bounded by
//   E(x) = (7.2e-7 + r) ||x|| C + r H + 6.2e-5 sqrt(d) (||x|| + C),  r = 6.1e-6 ceil(d / 16),
// C = max ||c||, H = max 0.5||c||^2 (scaled units).  If the best approximate score beats the second best by more than 2 E(x),
// the arg-max of the approximate scores IS the arg-max of the exact real-valued scores: the
// label is certain.  Otherwise (about 2 samples in 1000 on blob data) the sample is put on a
// queue of the workgroup in LDS and evaluated in plain fp32 after the last tile, one wave per
// entry: every lane takes the centroids lane, lane + 64, ... with feature-sequential fused
// multiply-adds from -0.5||c||^2, and the wave combines the results with the lowest index
// winning a tie.  A 32-sample column with several such samples, or one that finds the queue
// full, is redone as a whole in fp32 on the matrix cores instead.  Labels therefore meet the
// same bar as an all-fp32 evaluation (they can differ from it only where fp32's own rounding
// decides), and the sums are taken from the fp32 inputs in 64-bit fixed point exactly as in
// lloyd_mfma.hip.  Non-finite scores make a sample uncertain.
//
// fp64 inputs (TX = double) go through the same screen: the rows are rounded to fp32 as they
// arrive (one more 2^-24 per value, counted in the bound), the part of the bound that belongs to a
// centroid is kept per centroid (see PER_CENTROID in the kernel), and the samples the screen cannot
// certify - a few percent where two centroids share a blob, since the bound is relative to fp32
// roundings - are noted in a list of the workgroup and evaluated sixteen at a time on the fp64
// matrix cores after the last tile.  The sums are taken from the fp64 inputs, one rounding to the
// 64-bit fixed point per term.
//
// The same kernel without the update assigns labels only (kmx_assign_labels): there the scale
// comes from the centroids (any scale is correct, a sample that overflows fp16 merely fails the
// test) and each tile takes the norms of its samples itself.
//
// Work decomposition: as in lloyd_mfma.hip with two sample columns per lane.  Lane (j, h) of a
// wave owns features 16 s + 2 i + h (i < 8) of samples 2 j, 2 j + 1 of the wave's 64-sample
// tile: slot i of half-wave h is K index 8 h + i of K step s for both MFMA operands.
#include "lloyd_layout.h"
#include "lloyd_tail.h"

#include <type_traits>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef double v8d __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Error bound of one approximate score, in scaled units:
//   (SCR_ERR_SPLIT + r) ||x|| C + r H + SCR_ERR_ABS sqrt(d) (||x|| + C),
// r = SCR_ERR_ROUND * 51 * (K steps of 16 features): one ulp per addition of the accumulation
constexpr float SCR_ERR_SPLIT = 7.2e-7f;  // 3.01 * 2^-22, rounded up
// fp64 inputs reach the split through one rounding to fp32 (2^-24 relative, for x and for c): what
// the two fp16 parts leave out is then at most 1.25 * 2^-22 of a value instead of 2^-22, and the
// half norms in the scores are those of the rounded centroids (2^-23 relative)
constexpr float SCR_ERR_SPLIT_F64 = 9.6e-7f;  // 4.01 * 2^-22, rounded up
constexpr float SCR_ERR_HNEG_F64 = 1.2e-7f;   // 2^-23, rounded up
constexpr float SCR_ERR_ROUND = 1.2e-7f;  // 2^-23, rounded up
constexpr float SCR_ERR_ABS = 6.2e-5f;    // 2^-14, rounded up
// Scaled data lie in [2^(SCR_SCALE_EXP - 1), 2^SCR_SCALE_EXP): low enough for -0.5||c||^2 / SCR_HK_X1
// to stay inside fp16 for every d <= 31 (0.5 * 31 * 2^26 / 2^15 < 2^15), high enough for the
// absolute term of the bound to stay a few percent of the relative one.
constexpr int SCR_SCALE_EXP = 13;
// When the last K step has a feature slot to spare (d not a multiple of 16), -0.5||c||^2 rides in
// it instead of in the accumulator's start value: the samples carry the constant SCR_HK_X1 there
// (hi part; lo part zero) and the centroids the two fp16 parts of -0.5||c||^2 / SCR_HK_X1, so
// that hi*hi + lo*hi add it up to 2^-22 relative (SCR_ERR_HNEG), or 2^-14 * SCR_HK_X1 absolute
// should the lo part be flushed.  The accumulators then start from the constant zero: no read
// of sixteen start values per block and column, no registers for them.
constexpr float SCR_HK_X1 = 32768.0f;
constexpr float SCR_ERR_HNEG = 3.0e-7f;  // 2^-22 for the two-part value, 2^-24 for its fp32 original, rounded up
constexpr int SCR_GROUP = 8;  // accumulator registers per arg-max group
constexpr int SCR_REDO_COLUMN = 3;  // uncertain samples from which a 32-sample column is redone in fp32
// Words of the step's counter block in the workspace (`uncertain_count`): samples evaluated in
// fp32 by the running iteration, the same of the last finished one, and how the next step is
// to bring the sums up to date (written by the finalisation): 0 rebuild them, 1 correct them for
// the samples that change cluster, collected in the workgroup's list, 2 correct them tile by tile.
constexpr int SCR_WORD_DELTA = 2;
// Waves per workgroup (one workgroup per compute unit, or two of four waves).
#ifndef KMX_SCR_WAVES
#define KMX_SCR_WAVES 12
#endif
// Matrix-core and vector work of one wave interleaved (software pipeline over the centroid
// blocks); 0 restores blockwise scoring for comparison.
#ifndef KMX_SCR_PIPE
#define KMX_SCR_PIPE 1
#endif
// The winning group of a full tile is copied under an execution mask that the compare writes
// directly (one assembly block); 0 restores the compiler's save / branch / restore.
#ifndef KMX_SCR_CMPX
#define KMX_SCR_CMPX 1
#endif
constexpr int scr_waves(int nk) { return nk == 1 ? KMX_SCR_WAVES : (nk == 2 ? 4 : 8); }

struct ScreenLds {
    size_t off_afh, off_afl, off_hneg, off_ct, off_hx, off_ctx, off_hxx, off_qlist, off_queue, off_moved, total;
    int kp;       // centroids rounded up to a multiple of 64
    int ql_cap;   // fp64 inputs: samples the workgroup can note for evaluation (there is no queue then)
    int q_cap;    // entries of the queue of samples the screen could not certify
    int q_words;  // 32-bit words per entry: 16 nk feature values and the weight (in the input type), sample index, old label
    int m_cap;    // entries of the list of samples that change cluster (fused step)
};
constexpr int SCR_QUEUE_MAX = 256;
// fp64 inputs: a few percent of the samples of a blob that two centroids share fail a screen whose
// bound is relative to fp32 roundings, so the workgroup notes their indices (this many at most)
// and works them off sixteen at a time on the fp64 matrix cores, their rows gathered from memory
constexpr int SCR_QLIST_F64 = 4096;
// The list serves the iterations that correct the sums (at most one label in 24 changed in the
// iteration before: about n / 24 / workgroups entries); a tile that finds it full adds its
// changes on the spot.
constexpr int SCR_MOVED_MAX = 1024;
constexpr int SCR_MOVED_WORDS = 3;  // sample index, old label, new label
// LDS a workgroup may take: the compute unit has 160 KB; one workgroup of twelve waves per
// compute unit (one K step) or one of eight (three or four K steps: 256 registers per lane
// leave room for two waves per SIMD) can have nearly all of it, two workgroups of four waves
// (two K steps) half each.  Above 64 KB the kernel needs hipFuncAttributeMaxDynamicSharedMemorySize.
__host__ __device__ constexpr size_t scr_lds_max(int nk) { return nk == 2 ? 78 * 1024 : 156 * 1024; }
// esize: bytes of an input element (4, or 8: fp64 inputs keep an fp64 copy of the centroids and
// of their half norms for the samples the screen cannot certify)
__host__ __device__ inline ScreenLds screen_lds(int d, int k, int nk, bool update, int esize = 4) {
    ScreenLds s;
    // (an even number of centroid blocks: the scoring loop takes them in pairs; a block past
    // the last one holds padding only, whose scores are -inf)
    const size_t n_cb = (((size_t)(k + 31) / 32) + 1) & ~(size_t)1;
    // sums, cluster-major: per cluster the features, a spare word when d is odd, then the size
    const size_t acc = update ? (((size_t)(((d + 1) & ~1) + 1) * k * 8 + 15) & ~(size_t)15) : 0;
    s.off_afh = acc;
    s.off_afl = s.off_afh + n_cb * nk * 64 * 16;
    s.off_hneg = s.off_afl + n_cb * nk * 64 * 16;
    s.kp = (k + 63) & ~63;
    s.off_ct = s.off_hneg + n_cb * 32 * 4;             // fp32 centroids, (d, kp) (fp32 inputs only)
    s.off_hx = s.off_ct + (esize == 8 ? 0 : (size_t)d * s.kp * 4);  // fp32 (kp): 0.5||c||^2, +inf past k; fp64 inputs: the centroid's term of the bound
    s.off_ctx = (s.off_hx + (size_t)s.kp * 4 + 7) & ~(size_t)7;                   // fp64 inputs: centroids and half norms in fp64
    s.off_hxx = s.off_ctx + (esize == 8 ? (size_t)d * s.kp * 8 : 0);
    s.off_qlist = s.off_hxx + (esize == 8 ? (size_t)s.kp * 8 : 0);
    s.ql_cap = esize == 8 ? SCR_QLIST_F64 : 0;
    s.off_queue = s.off_qlist + (size_t)s.ql_cap * 4;
    // the queue takes what is left of the workgroup's LDS, up to SCR_QUEUE_MAX entries (none:
    // every uncertain sample is then handled where it turns up)
    s.q_words = (esize / 4) * (16 * nk + 1) + (esize == 8 ? 2 : 3);
    const size_t cap = scr_lds_max(nk);
    const size_t room = s.off_queue < cap ? (cap - s.off_queue) / ((size_t)s.q_words * 4) : 0;
    s.q_cap = esize == 8 ? 0 : (int)(room < (size_t)SCR_QUEUE_MAX ? room : (size_t)SCR_QUEUE_MAX);
    s.off_moved = s.off_queue + (size_t)s.q_cap * s.q_words * 4;
    const size_t room_m = (update && s.off_moved < cap) ? (cap - s.off_moved) / ((size_t)SCR_MOVED_WORDS * 4) : 0;
    s.m_cap = (int)(room_m < (size_t)SCR_MOVED_MAX ? room_m : (size_t)SCR_MOVED_MAX);
    s.total = s.off_moved + (size_t)s.m_cap * SCR_MOVED_WORDS * 4;
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

// 2^-a with max|x| * 2^-a in [2^(SCR_SCALE_EXP - 1), 2^SCR_SCALE_EXP) (1 for all-zero or non-finite data)
__device__ __forceinline__ float screen_scale(const float xmax) {
    return (xmax > 0.0f && xmax < kmx_inf<float>()) ? ldexpf(1.0f, SCR_SCALE_EXP - 1 - ilogbf(xmax)) : 1.0f;
}

// The fp16 pair of eight scaled values, as operand registers: hi = fp16(x * 2^-a) and
// lo = fp16(x * 2^-a - hi), each one mixed-precision fused multiply-add with a single rounding
// (the product with a power of two and the difference are exact); value i goes to half i % 2 of
// register i / 2.  `scale` is a scalar operand.
// Sixteen instructions in ONE statement: between separate statements the compiler pads every
// dependency on an assembly result with a wait state (it must assume a partial register
// write).  The real rule - a 16-bit write needs one instruction between it and a read of that
// register - is kept by the order: the four registers are written in rotation.  The closing
// s_nop gives a vector-ALU result the two wait states it needs before a matrix instruction may
// read it.
__device__ __forceinline__ void split_eight(const float v0, const float v1, const float v2, const float v3,
                                            const float v4, const float v5, const float v6, const float v7,
                                            const float scale, unsigned int (&hw)[4], unsigned int (&lw)[4]) {
    asm("v_fma_mixlo_f16 %0, %8, %16, 0\n\t"
        "v_fma_mixlo_f16 %1, %10, %16, 0\n\t"
        "v_fma_mixlo_f16 %2, %12, %16, 0\n\t"
        "v_fma_mixlo_f16 %3, %14, %16, 0\n\t"
        "v_fma_mixhi_f16 %0, %9, %16, 0\n\t"
        "v_fma_mixhi_f16 %1, %11, %16, 0\n\t"
        "v_fma_mixhi_f16 %2, %13, %16, 0\n\t"
        "v_fma_mixhi_f16 %3, %15, %16, 0\n\t"
        "v_fma_mixlo_f16 %4, %8, %16, -%0 op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixlo_f16 %5, %10, %16, -%1 op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixlo_f16 %6, %12, %16, -%2 op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixlo_f16 %7, %14, %16, -%3 op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %4, %9, %16, -%0 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %5, %11, %16, -%1 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %6, %13, %16, -%2 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %7, %15, %16, -%3 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "s_nop 1"
        : "=&v"(hw[0]), "=&v"(hw[1]), "=&v"(hw[2]), "=&v"(hw[3]), "=&v"(lw[0]), "=&v"(lw[1]), "=&v"(lw[2]),
          "=&v"(lw[3])
        : "v"(v0), "v"(v1), "v"(v2), "v"(v3), "v"(v4), "v"(v5), "v"(v6), "v"(v7), "s"(scale));
}

// Largest value over the 64 lanes of a wave (all of them active), the same in every lane: within
// rows of 16 lanes by four data-parallel steps (neighbour, other pair, other quad, other half of
// the row), then the four rows through scalar registers.
__device__ __forceinline__ unsigned int wave_umax(unsigned int v) {
    v = max(v, (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, true));   // quad_perm [1, 0, 3, 2]
    v = max(v, (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, true));   // quad_perm [2, 3, 0, 1]
    v = max(v, (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, true));  // row_half_mirror
    v = max(v, (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, true));  // row_mirror
    const unsigned int r0 = (unsigned int)__builtin_amdgcn_readlane((int)v, 0);
    const unsigned int r1 = (unsigned int)__builtin_amdgcn_readlane((int)v, 16);
    const unsigned int r2 = (unsigned int)__builtin_amdgcn_readlane((int)v, 32);
    const unsigned int r3 = (unsigned int)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(r0, r1), max(r2, r3));
}

__device__ __forceinline__ float scr_fma(float a, float b, float c) { return fmaf(a, b, c); }
__device__ __forceinline__ double scr_fma(double a, double b, double c) { return fma(a, b, c); }

// One column of 32 samples against all centroids in plain fp32 on the matrix cores
// (v_mfma_f32_32x32x2_f32 from -0.5||c||^2, lowest index wins a tie): the route for columns with
// several samples the screen cannot certify.  rows.v[8 s + i] = feature 16 s + 2 i + h of the
// lane's sample (NK K steps of 16 features); ct (d, kp) and hx (kp) are the fp32 centroids and
// half norms in LDS.
template <int NK>
struct ColumnRows {
    float v[8 * NK];
};
template <int NK>
__device__ __forceinline__ uint32_t redo_column_fp32(const ColumnRows<NK>& rows, const float* ct, const float* hx,
                                                  int n_cb, int d, int kp, int h, int j) {
    float bv = -kmx_inf<float>();
    int bc = 0x7fffffff;
    for (int cb = 0; cb < n_cb; ++cb) {
        v16f a;
#pragma unroll
        for (int r = 0; r < 16; ++r) a[r] = -hx[32 * cb + 8 * (r >> 2) + 4 * h + (r & 3)];
#pragma unroll
        for (int p = 0; p < 8 * NK; ++p) {
            const int p0 = 2 * p;  // features p0 + h; wave-uniform guard
            if (p0 < d) {
                const bool ok = p0 + h < d;
                const float af = ok ? ct[(p0 + h) * kp + 32 * cb + j] : 0.0f;
                const float xv = ok ? rows.v[p] : 0.0f;
                a = __builtin_amdgcn_mfma_f32_32x32x2f32(af, xv, a, 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r)  // increasing centroid index inside the lane
            if (a[r] > bv) {
                bv = a[r];
                bc = 32 * cb + 8 * (r >> 2) + 4 * h + (r & 3);
            }
    }
    const float ov = __shfl_xor(bv, 32, 64);
    const int oc = __shfl_xor(bc, 32, 64);
    if (ov > bv || (ov == bv && oc < bc)) bc = oc;
    if (bc == 0x7fffffff) bc = 0;  // no score compares: the reference's running arg-min keeps 0
    return (uint32_t)bc;
}

// INERTIA (labels only): the kernel also sums w_i ||x_i - c_label_i||^2 over its samples, in fp32
// per sample (the lane pair of a sample each takes every other feature) and fp64 across samples,
// into inertia_partial[blockIdx.x].  sample_weight may be null (unit weights).  The rows of a tile
// are then still needed at its end, so the next tile's are requested there and not while the
// tile is scored.
// TX: the type of X, the weights and the centroids.  fp64 inputs are rounded to fp32 where the rows
// arrive and are screened like fp32 ones (the bound counts that rounding); the samples the screen
// cannot certify are evaluated in fp64, and the sums are taken from the fp64 inputs.
template <typename TX, int NK, bool UPDATE, bool HK, bool INERTIA = false>
__global__ __launch_bounds__(64 * scr_waves(NK), NK == 1 ? scr_waves(1) / 4 : 2) void lloyd_screen_kernel(
    const TX* __restrict__ X_t, const TX* __restrict__ sample_weight,
    const TX* __restrict__ centroids_t, const uint32_t* __restrict__ labels_prev,
    uint32_t* __restrict__ labels, kmx_lloyd_status* __restrict__ status,
    const unsigned int* __restrict__ absmax, const int* __restrict__ q_exp,
    unsigned long long* __restrict__ gsum, uint32_t* __restrict__ uncertain_count,
    const float* __restrict__ norms, int64_t n, int d, int k, int vec_ok,
    double* __restrict__ inertia_partial, const LloydTail<TX> tail, const int fuse_tail) {
    static_assert(!(UPDATE && INERTIA), "the inertia rides with the labels-only kernel");
    constexpr bool F64 = sizeof(TX) == 8;
    static_assert(!(F64 && INERTIA), "fp64 inputs: labels and inertia are two calls");
    constexpr int ES = (int)sizeof(TX), FW = ES / 4;  // bytes and 32-bit words of an input element
    // (labels only: `status` is null outside the iteration loop)
    if ((UPDATE || status != nullptr) && status->state != KMX_RUNNING) return;

    constexpr int WAVES = scr_waves(NK), THREADS = 64 * WAVES;
    constexpr int MC = 2, TILE = 64;
    constexpr int G = SCR_GROUP, NG = 16 / SCR_GROUP;
    // HK: the feature slot that carries -0.5||c||^2: the last K index of the last K step (it
    // holds no feature, d being no multiple of 16), i.e. pair 7 of that step in the upper half-wave
    constexpr int SPARE = 16 * NK - 1;
    using Cols0 = std::integral_constant<int, 0>;  // column tags of the arg-max, column counts of a tile
    using Cols1 = std::integral_constant<int, 1>;
    using Cols2 = std::integral_constant<int, MC>;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int n_cb = (k + 31) >> 5;
    const int n_cbe = (n_cb + 1) & ~1;  // blocks in the operand arrays: an even number, padding at the end
    // Accumulators: cluster-major, acc_stride = d_even + 1 words per cluster: feature f in word f,
    // the cluster size in word d_even.  For odd d the word between them takes what the upper
    // half-wave adds for the feature that does not exist (never read), so that the update needs
    // neither a select nor a guard per lane; and with the cluster's words next to each other the
    // atomics of a lane differ by compile-time offsets only.
    const int d_even = (d + 1) & ~1;
    const int acc_stride = d_even + 1;
    const int items = acc_stride * k;
    const ScreenLds lay = screen_lds(d, k, NK, UPDATE, ES);
    unsigned long long* acc = reinterpret_cast<unsigned long long*>(smem_raw);  // [k][d_even + 1]
    v8h* afh = reinterpret_cast<v8h*>(smem_raw + lay.off_afh);                  // [n_cb][NK][64]
    v8h* afl = reinterpret_cast<v8h*>(smem_raw + lay.off_afl);
    float* hneg = reinterpret_cast<float*>(smem_raw + lay.off_hneg);            // [n_cb][2][16]
    float* ct = reinterpret_cast<float*>(smem_raw + lay.off_ct);                // [d][kp]
    float* hx = reinterpret_cast<float*>(smem_raw + lay.off_hx);                // [kp]
    // what the samples the screen cannot certify are evaluated with: the centroids and half norms
    // in the input type (fp32 inputs: the two arrays above)
    TX* ctx = F64 ? reinterpret_cast<TX*>(smem_raw + lay.off_ctx) : reinterpret_cast<TX*>(ct);   // [d][kp]
    TX* hxx = F64 ? reinterpret_cast<TX*>(smem_raw + lay.off_hxx) : reinterpret_cast<TX*>(hx);   // [kp]
    const int kp = lay.kp;
    // centroid value (f, c) as the screen takes it
    auto cval = [&](const int f, const int c) __attribute__((always_inline)) {
        if constexpr (F64) return (float)ctx[f * kp + c];
        else return ct[f * kp + c];
    };
    // Queue of the samples the screen could not certify, evaluated in fp32 by the whole
    // workgroup after the last tile: per entry the 16 NK feature values in feature order, the
    // weight, the sample index (QUEUE_FREE: never written) and the previous label.
    uint32_t* queue = reinterpret_cast<uint32_t*>(smem_raw + lay.off_queue);    // [q_cap][q_words]
    const int q_cap = lay.q_cap;
    // (features and weight in the input type, then two 32-bit words)
    constexpr int NKF = 16 * NK;
    constexpr int QW = FW * (NKF + 1) + (F64 ? 2 : 3), Q_WEIGHT = FW * NKF, Q_INDEX = FW * (NKF + 1),
                  Q_PREV = FW * (NKF + 1) + 1;
    constexpr uint32_t QUEUE_FREE = 0xffffffffu;
    // where a tile notes the index of an uncertain sample: the entry's index word, or (fp64
    // inputs) a list of indices
    uint32_t* qlist = reinterpret_cast<uint32_t*>(smem_raw + lay.off_qlist);
    const int note_cap = F64 ? lay.ql_cap : q_cap;
    auto noted = [&](const int slot) __attribute__((always_inline)) -> uint32_t& {
        return F64 ? qlist[slot] : queue[slot * QW + Q_INDEX];
    };
    __shared__ unsigned int queue_count;
    // Samples that change cluster while the sums are only corrected: (index, old label, new
    // label), their terms moved from the old to the new cluster after the last tile.
    uint32_t* moved = reinterpret_cast<uint32_t*>(smem_raw + lay.off_moved);    // [m_cap][3]
    const int m_cap = lay.m_cap;
    __shared__ unsigned int moved_count;
    __shared__ unsigned int changed_block;
    __shared__ unsigned int hmax_bits;
    __shared__ unsigned int uncertain_block;
    __shared__ unsigned long long wave_key[WAVES];  // INERTIA: one fp64 total per wave

    __shared__ unsigned int xmax_bits;
    __shared__ unsigned int tile_ticket;
    __shared__ int q_lds[68];  // binary points of the fixed-point sums: features (d <= 64), then the weights
    if (UPDATE && threadIdx.x <= d) q_lds[threadIdx.x] = q_exp[threadIdx.x];
    if (threadIdx.x == 0) {
        tile_ticket = WAVES;  // (the first WAVES tickets are the waves' own indices)
        changed_block = 0;
        queue_count = 0;
        moved_count = 0;
        hmax_bits = 0;
        uncertain_block = 0;
        xmax_bits = 0;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int wt_step = (int)gridDim.x * WAVES;
    const int wt_first = (int)blockIdx.x * WAVES + wave;
    const int n_fast = vec_ok ? (int)(n / TILE) : 0;
    // a last round of full tiles that is at most three quarters full is cut into
    // single-column tiles of 32 samples, spread over all the waves
    const int n_rounds = n_fast / wt_step;
    const int n_left = n_fast - n_rounds * wt_step;
    const bool halves = n_left > 0 && 4 * (int64_t)n_left <= 3 * (int64_t)wt_step;
    const int n_main = halves ? n_rounds * wt_step : n_fast;

    // Rows of the lane: feature 2 p + h for the pairs p = 8 s + i, row d - 1 where that feature
    // does not exist (the centroid operand is zero there, so any finite value will do).  A load
    // is the scalar address of the tile in row 0 plus a 32-bit byte offset of the lane that does
    // not change from tile to tile (d * n * 4 < 2^32 is a condition of this path): no vector
    // arithmetic and no branch per tile.
    // The loads are buffer loads: resource descriptor (the array) and tile offset in scalar
    // registers, the lane's offset in one vector register, so a load needs no address arithmetic.
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<TX*>(X_t), 0, (int)(uint32_t)((uint64_t)d * (uint64_t)n * (uint64_t)ES), 0x00020000);
    const __amdgpu_buffer_rsrc_t norms_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(UPDATE ? norms : reinterpret_cast<const float*>(X_t)), 0,
        (int)(uint32_t)((uint64_t)n * 4u), 0x00020000);
    const __amdgpu_buffer_rsrc_t pl_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(UPDATE ? labels_prev : labels), 0, (int)(uint32_t)((uint64_t)n * 4u), 0x00020000);
    const uint32_t own_off = (uint32_t)(MC * j + h) * 4u;  // the lane's own sample inside a tile
    uint32_t row_off[NK][8];
#pragma unroll
    for (int s = 0; s < NK; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = 16 * s + 2 * i + h;
            row_off[s][i] = (uint32_t)(f < d ? f : d - 1) * (uint32_t)n * (uint32_t)ES + (uint32_t)(MC * j * ES);
        }
    // (the spare slot's constant is put in where the rows are consumed: a select here would make
    // the wave wait for loads it has only just requested)
    auto load_rows_raw = [&](const int wt, auto& dst) __attribute__((always_inline)) {
        using TD = std::remove_reference_t<decltype(dst[0][0][0])>;  // float: for the screen; TX: for the sums
        const uint32_t tile = (uint32_t)wt * (uint32_t)(TILE * ES);  // wave-uniform byte offset in row 0
#pragma unroll
        for (int s = 0; s < NK; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if constexpr (F64) {
                    // two fp64 samples per load (rounded to fp32 for the screen)
                    const v4u q = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, row_off[s][i], tile, 0);
                    dst[s][i][0] = (TD)__hiloint2double((int)q[1], (int)q[0]);
                    dst[s][i][1] = (TD)__hiloint2double((int)q[3], (int)q[2]);
                } else {
                    const v2u q = __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, row_off[s][i], tile, 0);
                    dst[s][i][0] = __uint_as_float(q[0]);
                    dst[s][i][1] = __uint_as_float(q[1]);
                }
            }
    };
    // The rows, norm and previous label of a tile are requested while the tile before it
    // is scored (they are consumed at the very start of a tile, and nothing else of a tile
    // can start before them): a wave's own loads then cost it no waiting.
    float x[NK][8][MC];
    float norm_next = 0.0f;
    uint32_t pl_next = 0u;
    // fp64 inputs: the rows arrive as they are in memory (two samples per register quad) and are
    // rounded to fp32 when their tile starts - a conversion at the request would wait for the data
    v4u x_raw[F64 ? NK : 1][8];
    auto arrive = [&]() __attribute__((always_inline)) {
        if constexpr (F64) {
#pragma unroll
            for (int s = 0; s < NK; ++s)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    x[s][i][0] = (float)__hiloint2double((int)x_raw[s][i][1], (int)x_raw[s][i][0]);
                    x[s][i][1] = (float)__hiloint2double((int)x_raw[s][i][3], (int)x_raw[s][i][2]);
                }
        }
    };
    auto request = [&](const int wt_) __attribute__((always_inline)) {
        if (wt_ < n_main) {  // wave-uniform
            if constexpr (F64) {
                const uint32_t tile = (uint32_t)wt_ * (uint32_t)(TILE * ES);
#pragma unroll
                for (int s = 0; s < NK; ++s)
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        x_raw[s][i] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, row_off[s][i], tile, 0);
            } else {
                load_rows_raw(wt_, x);
            }
            if (UPDATE) {
                const uint32_t tile = (uint32_t)wt_ * (uint32_t)(TILE * 4);  // (4-byte arrays whatever the input type)
                norm_next = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(norms_rsrc, own_off, tile, 0));
                pl_next = __builtin_amdgcn_raw_buffer_load_b32(pl_rsrc, own_off, tile, 0);
            }
        }
    };
    // (more than one K step: the registers do not allow it, the tile's data are requested when it
    // starts; fp64 inputs of up to 32 features leave room for the raw rows of the next tile)
    constexpr bool AHEAD = NK == 1 || (F64 && NK == 2);
    // the wave's first tile: ticket = its index in the workgroup (in a scalar register: tile offsets are scalar operands)
    const int wt_start = __builtin_amdgcn_readfirstlane((int)blockIdx.x * WAVES + wave);

    // Everything below is derived from one pass over the centroids in memory: row f goes to
    // wave f % WAVES, all its loads are in flight together, and the fragments and norms are
    // then computed from the copy in LDS.
    {
        const int lane_ = threadIdx.x & 63, wave_ = threadIdx.x >> 6;
        // Labels only: max|x| is not known and any scale is a correct one (a sample that overflows
        // fp16 gives infinite or NaN scores, fails the test and is evaluated in fp32), so four
        // times max|c| stands in for it: samples lie around the centroids they are assigned to.
        // Fused step: the larger of max|x| and max|c|.  Centroids that are means of samples never
        // exceed max|x|; initial centroids from elsewhere can, and would overflow fp16 and leave
        // every sample uncertified.
        unsigned int my_absmax = (UPDATE && threadIdx.x < d) ? absmax[threadIdx.x] : 0u;
        for (int f = wave_; f < d; f += WAVES)
            for (int c = lane_; c < kp; c += 64) {
                const TX vx = c < k ? centroids_t[(size_t)f * k + c] : TX(0);
                const float v = (float)vx;
                if constexpr (F64) ctx[f * kp + c] = vx;
                else ct[f * kp + c] = v;
                my_absmax = max(my_absmax, __float_as_uint(fabsf(v) * (UPDATE ? 1.0f : 4.0f)));
            }
        // The wave's first tile is requested here, behind the loads of the centroids (loads
        // return in order): its rows travel while the operands are prepared.
        if (AHEAD) request(wt_start);
        __syncthreads();  // the shared words above are zero
        // (non-negative floats order like their bits)
        if (my_absmax != 0u) atomicMax(&xmax_bits, my_absmax);
    }
    __syncthreads();
    // 2^-a with max|x| * 2^-a in [2^(SCR_SCALE_EXP - 1), 2^SCR_SCALE_EXP) (1 for all-zero or non-finite data)
    const float xs = screen_scale(__uint_as_float(xmax_bits));
    // The four pieces of work below start at different waves (thread index rotated by a third,
    // a half, two thirds of the workgroup): each is a chain of LDS round trips too short to
    // fill the workgroup, and one after the other on the same threads they took 3.7 us.
    auto rotated = [&](const int by) { return (int)((threadIdx.x + THREADS - by) % THREADS); };
    // PER_CENTROID (fp64 inputs): the error bound of the score of centroid c,
    //   r (H_c + ||x|| ||c||) + split ||x|| ||c|| + (rounding of H_c) + absolute part,  H_c = 0.5||c||^2,
    // is kept per centroid instead of through max ||c|| and max H.  With ||x|| ||c|| <= 0.5||x||^2 + H_c
    // it is at most rho H_c + X, rho = 2 r + split + (rounding of H_c), X = (r + split) 0.5||x||^2 +
    // absolute part.  The scores start from -(1 - rho) H_c, which makes every computed score an
    // upper bound of the exact one up to X, and the winner b is certain when it leads by
    // 2 X + 2 rho H_b.  One far-away centroid (an initial centroid outside the data) then no longer
    // costs every sample its certificate.
    constexpr bool PER_CENTROID = F64;
    const float sigma = SCR_ERR_ROUND * 51.0f * (float)NK + SCR_ERR_SPLIT_F64;
    const float rho = sigma + SCR_ERR_ROUND * 51.0f * (float)NK + SCR_ERR_HNEG_F64 + (HK ? SCR_ERR_HNEG : 0.0f) +
                      SCR_ERR_ROUND;
    const float h_keep = PER_CENTROID ? 1.0f - rho : 1.0f;
    constexpr int ROT_HNEG = (THREADS / 3) & ~63, ROT_HX = THREADS / 2, ROT_ZERO = (2 * THREADS / 3) & ~63;
    // A operand: hi and lo parts of 32 centroids x 16 features per block and K step
    for (int idx = threadIdx.x; idx < n_cbe * NK * 64; idx += THREADS) {
        const int l = idx & 63;
        const int s = (idx >> 6) % NK;
        const int cb = (idx >> 6) / NK;
        const int c = 32 * cb + (l & 31);  // < kp; zero in ct from k on
        v8h hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = 16 * s + 2 * i + (l >> 5);
            float v = f < d ? cval(f, c) * xs : 0.0f;
            if (HK && f == SPARE) {
                // the spare slot: -0.5||c||^2 / SCR_HK_X1, summed exactly as for hneg below;
                // -inf for the padding past k, whose scores then never win
                v = -kmx_inf<float>();
                if (c < k) {
                    float sq = 0.0f;
#pragma unroll 8
                    for (int g = 0; g < d; ++g) {
                        const float cv = cval(g, c) * xs;
                        sq += cv * cv;
                    }
                    v = -(sq / 2.0f) * (1.0f / SCR_HK_X1) * h_keep;
                }
            }
            const _Float16 hb = (_Float16)v;
            hi[i] = hb;
            lo[i] = (_Float16)(v - (float)hb);
            if (HK && f == SPARE && !(c < k)) {
                // the -inf of the padding goes into the lo part alone: it then only meets the
                // sample's constant (hi part) and never a zero, which would give NaN
                hi[i] = (_Float16)0.0f;
                lo[i] = hb;
            }
        }
        afh[idx] = hi;
        afl[idx] = lo;
    }
    for (int idx = rotated(ROT_HNEG); idx < n_cbe * 32; idx += THREADS) {  // (-inf for the padding)
        const int cb = idx >> 5, hh = (idx >> 4) & 1, r = idx & 15;
        const int c = 32 * cb + 8 * (r >> 2) + 4 * hh + (r & 3);
        float v = -kmx_inf<float>();
        if (c < k) {
            float sq = 0.0f;
#pragma unroll 8
            for (int f = 0; f < d; ++f) {
                const float cv = cval(f, c) * xs;
                sq += cv * cv;
            }
            v = -(sq / 2.0f) * h_keep;
            // non-negative floats order like their bits; a NaN norm ends up as the maximum
            // and makes every sample uncertain
            atomicMax(&hmax_bits, __float_as_uint(sq / 2.0f));
            if constexpr (PER_CENTROID) hx[c] = 2.01f * rho * (sq / 2.0f);
        } else if (PER_CENTROID && c < kp) {
            hx[c] = 0.0f;
        }
        hneg[idx] = v;
    }
    // unscaled half norms for the samples the screen cannot certify
    for (int c = rotated(ROT_HX); c < kp; c += THREADS) {
        TX v = kmx_inf<TX>();
        if (c < k) {
            TX sq = TX(0);
#pragma unroll 8
            for (int f = 0; f < d; ++f) {
                const TX cv = ctx[f * kp + c];
                sq += cv * cv;
            }
            v = sq / TX(2);
        }
        hxx[c] = v;
    }
    if (UPDATE)
        for (int jx = rotated(ROT_ZERO); jx < items; jx += THREADS) acc[jx] = 0ull;
    for (int e = rotated(ROT_ZERO); e < note_cap; e += THREADS) noted(e) = QUEUE_FREE;
    for (int e = rotated(ROT_ZERO); e < m_cap; e += THREADS) moved[e * SCR_MOVED_WORDS] = QUEUE_FREE;
    __syncthreads();

    const unsigned int h4 = 4u * (unsigned int)h;
    const int n_wtiles = (int)((n + TILE - 1) / TILE);  // n < 2^29: tile and sample indices fit 32 bits
    unsigned int changed = 0;
    unsigned int n_uncertain = 0;  // wave-uniform
    double inertia_lane = 0.0;     // INERTIA: the lane's share of the weighted sum

    // uncertain when best - second <= thr_x * ||x|| + thr_0: twice the error bound, with a
    // margin for the rounding of the bound itself and of the hardware square root
    const float hmax = __uint_as_float(hmax_bits);
    const float cmax = sqrtf(2.0f * hmax), abs_term = SCR_ERR_ABS * sqrtf((float)d);
    const float round_term = SCR_ERR_ROUND * 51.0f * (float)NK;
    // (||x|| comes unscaled from kmx_lloyd_init, hence the factor xs)
    // (and a norm the kernel takes itself, from the scaled values: no factor)
    const float thr_x = 2.01f * (PER_CENTROID ? abs_term : (SCR_ERR_SPLIT + round_term) * cmax + abs_term) *
                        (UPDATE ? xs : 1.0f);
    // (per centroid: the term in ||x||^2)
    const float thr_xx = PER_CENTROID ? 2.01f * 0.5f * sigma * (UPDATE ? xs * xs : 1.0f) : 0.0f;
    const float thr_0 =
        PER_CENTROID ? 2.01f * (abs_term * cmax + (HK ? SCR_ERR_ABS * SCR_HK_X1 : 0.0f))
                     : 2.01f * (round_term * hmax + abs_term * cmax +
                                (HK ? SCR_ERR_HNEG * hmax + SCR_ERR_ABS * SCR_HK_X1 : 0.0f));
    // what a sample carries in the spare slot: its scaled value is SCR_HK_X1
    const float hk_x = SCR_HK_X1 / xs;
    // +inf the optimiser cannot see through (it would turn the median below into a maximum
    // with two canonicalising instructions in front)
    float pos_inf = kmx_inf<float>();
    asm volatile("" : "+s"(pos_inf));
    const float neg_inf = -kmx_inf<float>();
    // the scale as a scalar operand of the conversions
    const float xs_s = __uint_as_float((unsigned int)__builtin_amdgcn_readfirstlane((int)__float_as_uint(xs)));

    // Fused step: whether the sums are rebuilt from every sample (first iteration, or after one
    // that changed many labels) or only corrected for the samples whose label changes: the
    // fixed-point sums are integers, so taking a sample's terms off its old cluster and adding
    // them to the new one leaves exactly the sums a full pass would produce.
    const bool full_mode = UPDATE ? (uncertain_count[SCR_WORD_DELTA] == 0u) : false;  // wave-uniform
    // (corrected sums: whether the samples that move are few enough for the workgroup's list)
    const bool use_list = UPDATE ? (uncertain_count[SCR_WORD_DELTA] == 1u) : false;

    // One sample against every centroid in the input type, by the whole wave: lane l takes the
    // centroids l, l + 64, ... (fused multiply-adds in feature order from -0.5||c||^2, strict '>'
    // in increasing order), then the wave combines: the largest score, the lowest index among
    // the lanes that hold it.  `xat(f)`: feature f of the sample (wave-uniform).
    auto evaluate_sample = [&](auto&& xat) __attribute__((always_inline)) {
        TX bs = -kmx_inf<TX>();
        int bc = 0x7fffffff;
        // Two centroids per lane and pass, FB features at a time whose reads are in flight
        // together (past d the last row is read again and the sum left alone); the additions
        // stay in feature order.
        constexpr int FB = F64 ? 8 : 16;
        for (int c = lane; c < kp; c += 128) {
            const bool two = c + 64 < kp;  // wave-uniform: kp is a multiple of 64
            const int c1 = two ? c + 64 : c;
            const TX* col0 = ctx + c;
            const TX* col1 = ctx + c1;
            TX s0 = -hxx[c], s1 = -hxx[c1];
            if (F64 && !two) {
                // (a last odd pass: one chain; fp64 multiply-adds are not free)
                for (int f0 = 0; f0 < d; f0 += FB) {
                    TX xv[FB], a0[FB];
#pragma unroll
                    for (int i = 0; i < FB; ++i) {
                        const int f = f0 + i < d ? f0 + i : d - 1;  // wave-uniform
                        xv[i] = xat(f);
                        a0[i] = col0[f * kp];
                    }
#pragma unroll
                    for (int i = 0; i < FB; ++i) {
                        const TX t0 = scr_fma(xv[i], a0[i], s0);
                        s0 = f0 + i < d ? t0 : s0;
                    }
                }
            } else {
                for (int f0 = 0; f0 < d; f0 += FB) {
                    TX xv[FB], a0[FB], a1[FB];
#pragma unroll
                    for (int i = 0; i < FB; ++i) {
                        const int f = f0 + i < d ? f0 + i : d - 1;  // wave-uniform
                        xv[i] = xat(f);
                        a0[i] = col0[f * kp];
                        a1[i] = col1[f * kp];
                    }
#pragma unroll
                    for (int i = 0; i < FB; ++i) {
                        const TX t0 = scr_fma(xv[i], a0[i], s0), t1 = scr_fma(xv[i], a1[i], s1);
                        s0 = f0 + i < d ? t0 : s0;
                        s1 = f0 + i < d ? t1 : s1;
                    }
                }
            }
            if (s0 > bs) {
                bs = s0;
                bc = c;
            }
            if (two && s1 > bs) {
                bs = s1;
                bc = c1;
            }
        }
        if constexpr (F64) {
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const TX ov = __shfl_xor(bs, off, 64);
                const int oc = __shfl_xor(bc, off, 64);
                if (ov > bs || (ov == bs && oc < bc)) {
                    bs = ov;
                    bc = oc;
                }
            }
        } else {
            // (the score in an order-preserving integer form)
            const unsigned int sb = __float_as_uint((float)bs);
            const unsigned int ordered = sb ^ ((sb >> 31) ? 0xffffffffu : 0x80000000u);
            const unsigned int top = wave_umax(ordered);
            bc = (int)~wave_umax(ordered == top ? (unsigned int)~bc : 0u);
        }
        if (bc == 0x7fffffff) bc = 0;  // no score compares: the reference's running arg-min keeps 0
        return bc;
    };

    // One tile of NC sample columns per lane.  NC = 2: 64 samples, lane (j, h) scores samples
    // i0 and i0 + 1 (i0 = first + 2 j) against its half of every centroid block and, once the
    // two half-waves have exchanged their results, OWNS sample i0 + h (threshold test, label,
    // bookkeeping).  NC = 1: 32 samples, sample i0 = first + j, owned by the lower half-wave.
    // `load` fills the lane's rows x[s][i][t] = feature 16 s + 2 i + h of sample i0 + t (row
    // d - 1 where the feature does not exist: the centroid operand is zero there); it is called
    // again by the rare paths that need the fp32 values once more, so that they do not occupy
    // registers across the scoring.
    // `x`, `norm_in`, `pl_in`: the lane's rows, the owner's norm and previous label, loaded by the
    // caller (for full tiles: while the previous tile was being scored); `refill` is called once
    // they have been consumed and may load the next tile's into the same variables.
    // `put_label(label, whether the lane owns a sample in range, its index)` writes the label, at
    // once or (full tiles) together with the next tile's requests.
    auto process = [&](auto nc_tag, auto full_tag, auto&& load, auto&& refill, auto&& put_label,
                       float(&x)[NK][8][decltype(nc_tag)::value], float& norm_in, uint32_t& pl_in,
                       const int64_t i0) __attribute__((always_inline)) {
        constexpr int NC = decltype(nc_tag)::value;
        constexpr bool FULL = decltype(full_tag)::value;
        const int64_t my_idx = NC == 2 ? i0 + h : i0;
        const bool owner = NC == 2 ? true : h == 0;
        const bool in_range = FULL || my_idx < n;

        // the owner's norm and previous label
        // (taken here, with the rows: a wait for them further down would also wait for the label
        // store and the requests issued in between)
        float norm_mine = norm_in;
        uint32_t pl_mine = pl_in;
        asm volatile("" : "+v"(norm_mine), "+v"(pl_mine));
        // the A operands of the first centroid block, asked for ahead of the conversion below
        constexpr bool PIPELINED = KMX_SCR_PIPE && NK == 1 && decltype(nc_tag)::value == 2;
        v8h ah_first, al_first;
        if constexpr (PIPELINED) {
            ah_first = afh[lane];
            al_first = afl[lane];
        }

        // scaled fp16 split of the B operand (split_eight)
        v8h xh[NK][NC], xl[NK][NC];
        float own_sq[NC];  // labels only: the lane's part of ||x||^2, scaled
        {
            const float xs_sc = xs_s;  // (a local: operands of inline assembly must be the lambda's own)
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                own_sq[t] = 0.0f;
#pragma unroll
                for (int s = 0; s < NK; ++s) {
                    unsigned int hw[4], lw[4];
                    // the spare slot's constant (prefetched rows arrive without it)
                    float x7 = x[s][7][t];
                    if (HK && s == NK - 1) x7 = h ? hk_x : x7;
                    split_eight(x[s][0][t], x[s][1][t], x[s][2][t], x[s][3][t], x[s][4][t], x[s][5][t], x[s][6][t],
                                x7, xs_sc, hw, lw);
                    if (!UPDATE) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const float pv = (16 * s + 2 * i + h < d) ? x[s][i][t] * xs : 0.0f;
                            own_sq[t] = fmaf(pv, pv, own_sq[t]);
                        }
                    }
                    xh[s][t] = __builtin_bit_cast(v8h, make_uint4(hw[0], hw[1], hw[2], hw[3]));
                    xl[s][t] = __builtin_bit_cast(v8h, make_uint4(lw[0], lw[1], lw[2], lw[3]));
                }
            }
        }
        if constexpr (!INERTIA) refill();
        // (INERTIA: the owner's weight, wanted at the end of the tile)
        float w_mine = 1.0f;
        if constexpr (INERTIA) {
            if (sample_weight != nullptr && in_range && owner) w_mine = sample_weight[my_idx];
        }

        // Running arg-max by groups of G accumulator registers, plus the second largest of
        // the group maxima (the median of best, second and the new maximum).
        float best[NC], second[NC];
        unsigned int code[NC];
        // the winning group's registers, as pairs; whatever the registers hold until the first
        // group with a score above -inf overwrites them (no instruction spent on a reset)
        // (named scalars, not an array: they are written by inline assembly at several inlined
        // sites, and only scalars are certain to stay in registers then)
        static_assert(G == 8 && NC <= 2, "four register pairs per column, two columns");
        double s00, s01, s02, s03, s10, s11, s12, s13;
        asm volatile("" : "=v"(s00), "=v"(s01), "=v"(s02), "=v"(s03));
        asm volatile("" : "=v"(s10), "=v"(s11), "=v"(s12), "=v"(s13));
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            best[t] = neg_inf;
            second[t] = neg_inf;
            code[t] = 0;
        }

        // One arg-max group: registers g * G .. g * G + G - 1 of the accumulator `acc` of one
        // column (centroid block cb); bst / sec / cde and the four register pairs sa .. sd are
        // that column's running state.  g is a literal at every call.
        auto argmax_group_of = [&](const int cb, const int g, const v16f& av, float& bst, float& sec,
                                   unsigned int& cde, double& sa, double& sb, double& sc, double& sd)
                                   __attribute__((always_inline)) {
            const unsigned int cd = (unsigned int)(cb * NG + g);  // wave-uniform
            // The first read of the matrix-core result is an instruction the compiler
            // knows (the median of a, b and +inf is max(a, b)): it inserts the wait
            // states an MFMA result needs before a vector-ALU read, which it does not
            // do for operands of inline assembly.
            float m = __builtin_amdgcn_fmed3f(av[g * G], av[g * G + 1], pos_inf);
            static_assert(G == 8, "three three-operand maxima after the first pair");
            const v8d ad = __builtin_bit_cast(v8d, av);
            if constexpr (FULL && KMX_SCR_CMPX) {
                // One statement (see the conversion above).  Every lane of a full tile is active
                // here: the compare writes the execution mask itself, the copies of the winning
                // group run under it and the mask is set back to all lanes - no scalar save /
                // branch / restore around six instructions that nearly always run anyway (some
                // lane of 64 improves in almost every group).  Strict: the earlier group keeps a tie.
                asm volatile(
                    "v_max3_f32 %[m], %[m], %[v2], %[v3]\n\t"
                    "v_max3_f32 %[m], %[m], %[v4], %[v5]\n\t"
                    "v_max3_f32 %[m], %[m], %[v6], %[v7]\n\t"
                    "v_med3_f32 %[sec], %[bst], %[sec], %[m]\n\t"
                    "v_cmpx_gt_f32_e32 %[m], %[bst]\n\t"
                    "v_mov_b32 %[bst], %[m]\n\t"
                    "v_mov_b32 %[cde], %[cd]\n\t"
                    "v_mov_b64 %[sa], %[a0]\n\t"
                    "v_mov_b64 %[sb], %[a1]\n\t"
                    "v_mov_b64 %[sc], %[a2]\n\t"
                    "v_mov_b64 %[sd], %[a3]\n\t"
                    "s_mov_b64 exec, -1"
                    : [m] "+v"(m), [sec] "+v"(sec), [bst] "+v"(bst), [cde] "+v"(cde), [sa] "+v"(sa), [sb] "+v"(sb),
                      [sc] "+v"(sc), [sd] "+v"(sd)
                    : [v2] "v"(av[g * G + 2]), [v3] "v"(av[g * G + 3]), [v4] "v"(av[g * G + 4]), [v5] "v"(av[g * G + 5]),
                      [v6] "v"(av[g * G + 6]), [v7] "v"(av[g * G + 7]), [cd] "s"(cd), [a0] "v"(ad[g * 4]),
                      [a1] "v"(ad[g * 4 + 1]), [a2] "v"(ad[g * 4 + 2]), [a3] "v"(ad[g * 4 + 3])
                    : "vcc");
                return;
            }
            // (one statement: see the conversion above)
            asm("v_max3_f32 %0, %0, %2, %3\n\t"
                "v_max3_f32 %0, %0, %4, %5\n\t"
                "v_max3_f32 %0, %0, %6, %7\n\t"
                "v_med3_f32 %1, %8, %1, %0"
                : "+v"(m), "+v"(sec)
                : "v"(av[g * G + 2]), "v"(av[g * G + 3]), "v"(av[g * G + 4]), "v"(av[g * G + 5]), "v"(av[g * G + 6]),
                  "v"(av[g * G + 7]), "v"(bst));
            // strict: the earlier group keeps a tie
            if (m > bst) {
                bst = m;
                cde = cd;
                asm volatile("v_mov_b64 %0, %1" : "+v"(sa) : "v"(ad[g * 4]));
                asm volatile("v_mov_b64 %0, %1" : "+v"(sb) : "v"(ad[g * 4 + 1]));
                asm volatile("v_mov_b64 %0, %1" : "+v"(sc) : "v"(ad[g * 4 + 2]));
                asm volatile("v_mov_b64 %0, %1" : "+v"(sd) : "v"(ad[g * 4 + 3]));
            }
        };
        auto argmax_group = [&](const int cb, auto g_tag, auto t_tag, const v16f& av) __attribute__((always_inline)) {
            constexpr int g = decltype(g_tag)::value, t = decltype(t_tag)::value;
            if constexpr (t == 0)
                argmax_group_of(cb, g, av, best[0], second[0], code[0], s00, s01, s02, s03);
            else
                argmax_group_of(cb, g, av, best[NC - 1], second[NC - 1], code[NC - 1], s10, s11, s12, s13);
        };
        using G0 = std::integral_constant<int, 0>;
        using G1 = std::integral_constant<int, 1>;
        static_assert(NG == 2, "two arg-max groups per accumulator");
        auto load_hneg = [&](const int cb, v16f& hv) __attribute__((always_inline)) {
            const float4* hp = reinterpret_cast<const float4*>(hneg + cb * 32 + h * 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 v4 = hp[q];
                hv[4 * q] = v4.x;
                hv[4 * q + 1] = v4.y;
                hv[4 * q + 2] = v4.z;
                hv[4 * q + 3] = v4.w;
            }
        };

        if constexpr (PIPELINED) {
            // Software pipeline over the stages (block cb, column t), t fastest: while the vector
            // ALU works through the scores of one stage, the matrix core already forms those of
            // the next (the other column's accumulator), one MFMA of its chain of three issued
            // ahead of each arg-max group.  fp16 MFMAs run beside vector instructions on this
            // hardware, but only if a wave has both kinds to issue: with all MFMAs of a block
            // first and all of its arg-max after, the waves of a SIMD fall into step and the two
            // units take turns.
            v16f a0, a1, hv;  // hv: the accumulators' start, -0.5||c||^2 of the block or (HK) zero
            v8h ahA, alA, ahB, alB;  // A operands of the block at hand and of the next one
            ahA = ah_first;
            alA = al_first;
            if constexpr (HK) {
#pragma unroll
                for (int r = 0; r < 16; ++r) hv[r] = 0.0f;
            } else {
                load_hneg(0, hv);
            }
            a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahA, xh[0][0], hv, 0, 0, 0);
            a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahA, xl[0][0], a0, 0, 0, 0);
            a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(alA, xh[0][0], a0, 0, 0, 0);
            // stages (cb, 0) and (cb, 1); (ahC, alC) hold block cb, (ahN, alN) receive block cb + 1
            // when there is one (MORE)
            auto block_pair = [&](auto more_tag, const int cb, const v8h& ahC, const v8h& alC, v8h& ahN, v8h& alN)
                                  __attribute__((always_inline)) {
                constexpr bool MORE = decltype(more_tag)::value;
                a1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahC, xh[0][1], hv, 0, 0, 0);
                if constexpr (MORE) {
                    ahN = afh[(cb + 1) * 64 + lane];
                    alN = afl[(cb + 1) * 64 + lane];
                }
                argmax_group(cb, G0{}, Cols0{}, a0);
                if constexpr (MORE && !HK) load_hneg(cb + 1, hv);  // its last reader, the MFMA above, has long finished
                a1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahC, xl[0][1], a1, 0, 0, 0);
                argmax_group(cb, G1{}, Cols0{}, a0);
                a1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(alC, xh[0][1], a1, 0, 0, 0);
                if constexpr (MORE) a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahN, xh[0][0], hv, 0, 0, 0);
                argmax_group(cb, G0{}, Cols1{}, a1);
                if constexpr (MORE) a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahN, xl[0][0], a0, 0, 0, 0);
                argmax_group(cb, G1{}, Cols1{}, a1);
                if constexpr (MORE) a0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(alN, xh[0][0], a0, 0, 0, 0);
            };
            // (n_cbe is even: an odd number of real blocks is followed by one of padding, whose
            // scores are -inf; one straight-line tail, so that no registers change place at a join)
            int cb = 0;
            for (; cb + 2 < n_cbe; cb += 2) {
                block_pair(std::true_type{}, cb, ahA, alA, ahB, alB);
                block_pair(std::true_type{}, cb + 1, ahB, alB, ahA, alA);
            }
            block_pair(std::true_type{}, cb, ahA, alA, ahB, alB);
            block_pair(std::false_type{}, cb + 1, ahB, alB, ahA, alA);
        } else {
            for (int cb = 0; cb < n_cb; ++cb) {
                v16f a[NC], hv;
                if constexpr (HK) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) hv[r] = 0.0f;
                } else {
                    load_hneg(cb, hv);
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
                argmax_group(cb, G0{}, Cols0{}, a[0]);
                if constexpr (NC == 2) argmax_group(cb, G0{}, Cols1{}, a[1]);
                argmax_group(cb, G1{}, Cols0{}, a[0]);
                if constexpr (NC == 2) argmax_group(cb, G1{}, Cols1{}, a[1]);
            }
        }

        // Per column and half-wave: position inside the winning group and the second largest
        // inside it.
        float sec_c[NC];
        unsigned int cen_c[NC];
#pragma unroll
        for (int t = 0; t < NC; ++t) {
            float sv[G];
#pragma unroll
            for (int r = 0; r < G / 2; ++r) {
                const double pair = t == 0 ? (r == 0 ? s00 : r == 1 ? s01 : r == 2 ? s02 : s03)
                                           : (r == 0 ? s10 : r == 1 ? s11 : r == 2 ? s12 : s13);
                const float2 pr = __builtin_bit_cast(float2, pair);
                sv[2 * r] = pr.x;
                sv[2 * r + 1] = pr.y;
            }
            // The lowest register equal to the best is the label's.  Register r of group g of
            // block b holds centroid 32 b + 16 g + 8 (r / 4) + 4 h + r % 4 (G = 8): the chain
            // selects 8 (r / 4) + r % 4 directly.
            static_assert(G == 8 && NG == 2, "centroid index below assumes two groups of eight");
            unsigned int pos = 8 * ((G - 1) >> 2) + ((G - 1) & 3);
#pragma unroll
            for (int r = G - 2; r >= 0; --r)
                pos = (sv[r] == best[t]) ? (unsigned int)(8 * (r >> 2) + (r & 3)) : pos;
            // Second largest of the eight (equal to the largest if that occurs twice), by a
            // tournament of (largest, second) pairs: triples give max3 / med3, and two pairs
            // merge into (max(m, m'), max3(min(m, m'), s, s')).
            // (temporaries %1 .. %4; one statement: see the conversion above)
            float tA, tB, tC, tD;
            asm("v_max3_f32 %1, %5, %6, %7\n\t"     // mA
                "v_max3_f32 %2, %8, %9, %10\n\t"    // mB
                "v_med3_f32 %3, %5, %6, %7\n\t"     // sA
                "v_med3_f32 %4, %8, %9, %10\n\t"    // sB
                "v_min_f32 %0, %1, %2\n\t"          // min(mA, mB)
                "v_max_f32 %1, %1, %2\n\t"          // mAB
                "v_max3_f32 %0, %0, %3, %4\n\t"     // sAB
                "v_max_f32 %2, %11, %12\n\t"        // mC
                "v_min_f32 %3, %11, %12\n\t"        // sC
                "v_min_f32 %1, %1, %2\n\t"          // min(mAB, mC)
                "v_max3_f32 %0, %1, %0, %3\n\t"     // second largest of the eight
                "v_max_f32 %0, %0, %13"               // or of the other groups' maxima
                : "=&v"(sec_c[t]), "=&v"(tA), "=&v"(tB), "=&v"(tC), "=&v"(tD)
                : "v"(sv[0]), "v"(sv[1]), "v"(sv[2]), "v"(sv[3]), "v"(sv[4]), "v"(sv[5]), "v"(sv[6]), "v"(sv[7]),
                  "v"(second[t]));
            cen_c[t] = (code[t] << 4) + pos + h4;
        }

        // The half-waves exchange results: one register swap per quantity gives the lower
        // half-wave both halves' results for column 0 and the upper one those for column 1
        // (NC = 1: both get column 0), so that each lane finishes ONE sample.  No LDS traffic
        // that would queue behind the accumulator atomics.
        const auto bb = __builtin_amdgcn_permlane32_swap(__float_as_uint(best[0]), __float_as_uint(best[NC - 1]),
                                                         false, false);
        const auto ss = __builtin_amdgcn_permlane32_swap(__float_as_uint(sec_c[0]), __float_as_uint(sec_c[NC - 1]),
                                                         false, false);
        const auto cc = __builtin_amdgcn_permlane32_swap(cen_c[0], cen_c[NC - 1], false, false);
        const float b_lo = __uint_as_float(bb[0]), b_hi = __uint_as_float(bb[1]);
        // second best over both halves: the loser of the two bests or a half's own second
        float s2, b;
        asm("v_min_f32 %0, %2, %3\n\t"
            "v_max_f32 %1, %2, %3\n\t"
            "v_max3_f32 %0, %0, %4, %5"
            : "=&v"(s2), "=&v"(b)
            : "v"(b_lo), "v"(b_hi), "v"(__uint_as_float(ss[0])), "v"(__uint_as_float(ss[1])));
        // the lower centroid index wins a tie between the halves
        const bool take_hi = b_hi > b_lo || (b_hi == b_lo && cc[1] < cc[0]);
        uint32_t lab_mine = take_hi ? cc[1] : cc[0];
        if (!UPDATE) {
            const auto qq = __builtin_amdgcn_permlane32_swap(__float_as_uint(own_sq[0]),
                                                             __float_as_uint(own_sq[NC - 1]), false, false);
            norm_mine = sqrtf(__uint_as_float(qq[0]) + __uint_as_float(qq[1]));
        }
        // written so that a NaN anywhere makes the sample uncertain
        float thr = fmaf(thr_x, norm_mine, thr_0);
        if constexpr (PER_CENTROID)  // (an index below kp whatever the scores)
            thr = fmaf(fmaf(thr_xx, norm_mine, thr_x), norm_mine, thr_0) + hx[lab_mine];
#ifdef KMX_SCR_NO_UNSURE
        const bool unsure_mine = false;
#else
        const bool unsure_mine = !(b - s2 > thr) && in_range && owner;
#endif

        // Samples the screen cannot certify go to the workgroup's queue (their label below is
        // provisional and they take no part in the sums here); the queue is worked off in plain
        // fp32 after the last tile, by all waves alike, so that no wave is held up by the samples
        // it happens to meet.  A column with several such samples (ties between duplicate
        // centroids, degenerate data), or one that finds the queue full, is instead redone as a
        // whole in fp32 on the matrix cores, which bounds the cost of a tile at about three times
        // the usual one however many samples fail the screen.
        bool queued_mine = false;
        const unsigned long long todo_all = __ballot(unsure_mine);  // bit 32 t + j: sample j of column t
        if (__builtin_expect(todo_all != 0ull, 0)) {                // cold: spills belong in here
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                const unsigned int todo = (unsigned int)(todo_all >> (32 * t));  // wave-uniform
                if (todo == 0u) continue;
                const int n_todo = __popc(todo);
                n_uncertain += (unsigned int)n_todo;
                // (fp64 inputs have no matrix-core route for a whole column: everything goes to the queue)
                bool redo = !F64 && n_todo >= SCR_REDO_COLUMN;
                unsigned int base = 0;
                if (!redo) {
                    if (lane == 0) base = atomicAdd(&queue_count, (unsigned int)n_todo);
                    base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
                    redo = base + (unsigned int)n_todo > (unsigned int)note_cap;
                }
                const bool col_mine = NC == 2 ? h == t : true;  // whether the lane's own sample is in column t
                if (redo && F64) {
                    // queue full: the wave evaluates the column's uncertain samples at once, one
                    // after the other, its features straight from memory
                    for (unsigned int rest = todo; rest != 0u; rest &= rest - 1u) {
                        const int jj = __builtin_ctz(rest);  // wave-uniform
                        const int64_t smp = i0 - (NC == 2 ? MC * j : j) + (NC == 2 ? MC * jj + t : jj);
                        const uint32_t r = (uint32_t)evaluate_sample(
                            [&](const int f) __attribute__((always_inline)) { return X_t[(size_t)f * n + smp]; });
                        if (col_mine && j == jj) lab_mine = r;
                    }
                } else if (redo) {
                    if constexpr (!F64) {
                        float xr[NK][8][NC];
                        load(xr);
                        ColumnRows<NK> rows;
#pragma unroll
                        for (int s = 0; s < NK; ++s)
#pragma unroll
                            for (int i = 0; i < 8; ++i) rows.v[8 * s + i] = xr[s][i][t];
                        const uint32_t r = redo_column_fp32<NK>(rows, ct, hx, n_cb, d, kp, h, j);
                        if (col_mine) lab_mine = r;
                    }
                } else if ((todo >> j) & 1u) {  // both lanes of the sample
                    // (the index alone: the entry's features, weight and previous label are
                    // fetched after the last tile, all entries of the workgroup at once, so
                    // that the tile does not wait for a second read of its rows)
                    const unsigned int slot = base + (unsigned int)__popc(todo & ((1u << j) - 1u));
                    if (h == 0) noted((int)slot) = (uint32_t)(i0 + t);
                    if (col_mine) queued_mine = true;
                }
            }
        }

        put_label(lab_mine, in_range && owner, my_idx);

        if constexpr (INERTIA) {
            // both columns' labels in every lane: the lane takes its features of both samples,
            // in feature order from an fp32 copy of the centroids in LDS; a sample's two halves
            // are added by its owner.  Queued samples are added when the queue is worked off.
            uint32_t lab[NC];
            const auto ll = __builtin_amdgcn_permlane32_swap(lab_mine, lab_mine, false, false);
            lab[0] = ll[0];
            if (NC == 2) lab[NC - 1] = ll[1];
            float part[NC];
#pragma unroll
            for (int t = 0; t < NC; ++t) {
                part[t] = 0.0f;
                const float* ccol = ct + (lab[t] < (uint32_t)kp ? lab[t] : 0u);
#pragma unroll
                for (int s = 0; s < NK; ++s)
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int f = 16 * s + 2 * i + h;
                        if (f < d) {
                            const float diff = x[s][i][t] - ccol[f * kp];
                            part[t] = fmaf(diff, diff, part[t]);
                        }
                    }
            }
            const auto qq = __builtin_amdgcn_permlane32_swap(__float_as_uint(part[0]), __float_as_uint(part[NC - 1]),
                                                             false, false);
            const float sq_mine = __uint_as_float(qq[0]) + __uint_as_float(qq[1]);
            if (in_range && owner && !queued_mine) inertia_lane += (double)(sq_mine * w_mine);
            refill();
        }

        if (UPDATE) {
            const bool counted_mine = in_range && owner && !queued_mine;
            const bool chg_mine = counted_mine && pl_mine != lab_mine;
            changed += chg_mine ? 1u : 0u;
            // which samples the sums have to hear of: all of them when the sums are rebuilt,
            // those that change cluster otherwise (bit 32 t + j: sample j of column t)
            const unsigned long long act_all = __ballot(full_mode ? counted_mine : chg_mine);
            // Sums only corrected: the few samples that move go on the workgroup's list and are
            // dealt with after the last tile (one thread per sample and feature, all reads in
            // flight together); a tile does not read its rows a second time for them.
            bool listed = false;  // wave-uniform
            if (act_all != 0ull && use_list && m_cap > 0) {
                const unsigned int n_act = (unsigned int)__popcll(act_all);
                unsigned int base = 0;
                if (lane == 0) base = atomicAdd(&moved_count, n_act);
                base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
                listed = base + n_act <= (unsigned int)m_cap;
                if (listed && chg_mine) {
                    uint32_t* entry =
                        moved + (base + (unsigned int)__popcll(act_all & ((1ull << lane) - 1ull))) * SCR_MOVED_WORDS;
                    entry[1] = pl_mine;
                    entry[2] = lab_mine;
                    entry[0] = (uint32_t)my_idx;
                }
            }
            if (act_all != 0ull && !listed) {
                TX xr[NK][8][NC];
                load(xr);
                // both columns' labels in every lane (the lane adds its features of both samples)
                uint32_t lab[NC], pl[NC];
                const auto ll = __builtin_amdgcn_permlane32_swap(lab_mine, lab_mine, false, false);
                const auto pp = __builtin_amdgcn_permlane32_swap(pl_mine, pl_mine, false, false);
                lab[0] = ll[0];
                pl[0] = pp[0];
                if (NC == 2) {
                    lab[NC - 1] = ll[1];
                    pl[NC - 1] = pp[1];
                }
#pragma unroll
                for (int t = 0; t < NC; ++t) {
                    const unsigned int act_col = (unsigned int)(act_all >> (32 * t));  // wave-uniform
                    if (act_col == 0u) continue;
                    const bool act = (act_col >> j) & 1u;
                    // samples past the end and samples that stay put are not in the mask
                    const double wd = act ? (double)sample_weight[i0 + t] : 0.0;  // (fp64 inputs: exact)
                    unsigned long long* to = acc + lab[t] * (uint32_t)acc_stride + h;    // word h of the new cluster
                    unsigned long long* from = acc + pl[t] * (uint32_t)acc_stride + h;   // and of the old one
#pragma unroll
                    for (int s = 0; s < NK; ++s)
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const int p0 = 16 * s + 2 * i;  // the pair's even feature
                            if (p0 < d) {                   // wave-uniform
                                // (odd d, last pair: the upper half-wave adds to the spare word)
                                const double magic = fix_magic(q_lds[p0 + h]);
                                // x * w is exact in fp64; one rounding, to a multiple of 2^-q
                                const double v = fma((double)xr[s][i][t], wd, magic);
                                const unsigned long long term = to_fixed_q(v, magic);
                                if (act) {
                                    atomicAdd(to + p0, term);
                                    if (!full_mode) atomicSub(from + p0, term);
                                }
                            }
                        }
                    if (h == 0 && act) {
                        const double magic_w = fix_magic(q_lds[d]);
                        const unsigned long long term = to_fixed_q(wd + magic_w, magic_w);
                        atomicAdd(to + d_even, term);
                        if (!full_mode) atomicSub(from + d_even, term);
                    }
                }
            }
        }
    };

    auto load_rows = [&](const int wt, auto& dst) __attribute__((always_inline)) {
        using TD = std::remove_reference_t<decltype(dst[0][0][0])>;
        load_rows_raw(wt, dst);
        if (HK) {
            // the spare slot carries the constant whose scaled value is SCR_HK_X1
#pragma unroll
            for (int t = 0; t < MC; ++t) dst[NK - 1][7][t] = h ? (TD)hk_x : dst[NK - 1][7][t];
        }
    };

    // The workgroup's full tiles (tile WAVES * blockIdx.x + q % WAVES of round q / WAVES) are
    // handed out through a ticket counter in LDS: the waves of a workgroup do not advance at
    // the same pace, and with fixed shares the fastest would wait a fifth of the time for the
    // slowest at the end.  The next ticket is drawn before the current tile is worked on.
    if (n_main > 0) {
        auto draw = [&]() __attribute__((always_inline)) {
            unsigned int ticket = 0;
            if (lane == 0) ticket = atomicAdd(&tile_ticket, 1u);
            return ticket;  // valid in lane 0
        };
        auto tile_of = [&](const unsigned int ticket_) __attribute__((always_inline)) {
            const int q = __builtin_amdgcn_readfirstlane((int)ticket_);
            return (int)blockIdx.x * WAVES + q % WAVES + (q / WAVES) * wt_step;
        };
        // The labels of a tile are written when the NEXT tile has started, just ahead of the
        // requests for the tile after it: the wave waits for everything it has in flight when it
        // starts a tile (stores count like loads), and a store issued at the end of a tile would
        // make it wait for that store's acknowledgement every time.
        uint32_t lab_pending = 0u;
        int wt_pending = -1;  // wave-uniform; -1: nothing to write
        uint32_t* const labels_lane = labels + own_off / 4u;
        auto write_pending = [&]() __attribute__((always_inline)) {
            if (wt_pending >= 0) labels_lane[(int64_t)wt_pending * TILE] = lab_pending;
        };
        int wt = wt_start;
        while (wt < n_main) {  // every wave gets out: the counter only grows
            const int wt_next = tile_of(draw());
            const int64_t i0 = (int64_t)wt * TILE + MC * j;
            const int wt_now = wt;
            if (!AHEAD) request(wt_now);
            arrive();
            uint32_t lab_now = 0u;
            process(
                Cols2{}, std::true_type{},
                [&](auto& xr) __attribute__((always_inline)) { load_rows(wt_now, xr); },
                [&]() __attribute__((always_inline)) {
                    write_pending();
                    if (AHEAD) request(wt_next);
                },
                [&](const uint32_t lab, bool, int64_t) __attribute__((always_inline)) { lab_now = lab; },
                x, norm_next, pl_next, i0);
            lab_pending = lab_now;
            wt_pending = wt_now;
            wt = wt_next;
        }
        write_pending();
    }
    auto put_now = [&](const uint32_t lab, const bool mine, const int64_t idx) __attribute__((always_inline)) {
        if (mine) labels[idx] = lab;
    };
    // scalar loads of the lane's rows (row d - 1 where the feature does not exist)
    auto load_scalar = [&](auto nc_tag, const int64_t i0, auto& dst) __attribute__((always_inline)) {
        using TD = std::remove_reference_t<decltype(dst[0][0][0])>;
        constexpr int NC = decltype(nc_tag)::value;
#pragma unroll
        for (int s = 0; s < NK; ++s)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int f = 16 * s + 2 * i + h;
                const TX* row = X_t + (size_t)(f < d ? f : d - 1) * n;
                const TD absent = (HK && f == SPARE) ? (TD)hk_x : TD(0);  // the spare slot, or no feature at all
#pragma unroll
                for (int t = 0; t < NC; ++t) dst[s][i][t] = f < d ? (i0 + t < n ? (TD)row[i0 + t] : TD(0)) : absent;
            }
    };
    if (halves) {
        // single-column tile q of the left-over tiles: samples [n_main * TILE + 32 q, + 32)
        for (int q = wt_first; q < MC * n_left; q += wt_step) {
            const int64_t i0 = (int64_t)n_main * TILE + 32 * q + j;
            float x[NK][8][1];
            load_scalar(Cols1{}, i0, x);
            float norm_now = UPDATE ? norms[i0] : 0.0f;
            uint32_t pl_now = UPDATE ? labels_prev[i0] : 0u;
            process(
                Cols1{}, std::true_type{},
                [&](auto& xr) __attribute__((always_inline)) { load_scalar(Cols1{}, i0, xr); }, [] {},
                put_now, x, norm_now, pl_now, i0);
        }
    }
    // The rest: a partial last tile, or every tile when vector accesses are not legal
    for (int wt = n_fast + wt_first; wt < n_wtiles; wt += wt_step) {
        const int64_t i0 = (int64_t)wt * TILE + MC * j;
        float x[NK][8][MC];
        load_scalar(Cols2{}, i0, x);
        const bool mine_exists = i0 + h < n;
        float norm_now = (UPDATE && mine_exists) ? norms[i0 + h] : 0.0f;
        uint32_t pl_now = (UPDATE && mine_exists) ? labels_prev[i0 + h] : 0u;
        process(
            Cols2{}, std::false_type{},
            [&](auto& xr) __attribute__((always_inline)) { load_scalar(Cols2{}, i0, xr); }, [] {},
            put_now, x, norm_now, pl_now, i0);
    }

    // The samples noted by the tiles.
    __syncthreads();  // lists complete; provisional labels have reached memory
    const int n_noted = (int)min(queue_count, (unsigned int)note_cap);
    if constexpr (!F64) {
        // one wave per entry of the queue (evaluate_sample), once the entries are filled in
        const int n_queued = n_noted;
        // The queue's entries: features in feature order (zero past d) and the weight in the input
        // type, then the index and the previous label.  Thread (entry, slot) fetches one value,
        // eight per thread and pass with all their reads in flight together (a loop of one load and
        // one store per pass would take a trip to memory per pass).
        {
            constexpr int SLOTS = NKF + 2;  // features, weight, (index, previous label)
            constexpr int U = 8;
            const int total = n_queued * SLOTS;
            for (int first = 0; first < total; first += U * THREADS) {
                TX val[U];
                uint32_t idx[U], prv[U];
                int at[U];  // first word of the value in the queue; -1: nothing to store
                bool pair[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int item = first + u * THREADS + (int)threadIdx.x;
                    at[u] = -1;
                    pair[u] = false;
                    val[u] = TX(0);
                    idx[u] = prv[u] = 0u;
                    if (item < total) {
                        const int e = item / SLOTS, sl = item - e * SLOTS;
                        const uint32_t sample = noted(e);
                        if (sl == NKF + 1) {
                            // (QUEUE_FREE: a slot reserved and never written; the index word says so)
                            at[u] = e * QW + Q_INDEX;
                            pair[u] = true;
                            idx[u] = sample;
                            if (UPDATE && sample != QUEUE_FREE) prv[u] = labels_prev[sample];
                        } else if (sample != QUEUE_FREE) {
                            at[u] = e * QW + FW * sl;
                            if (sl < NKF) {
                                if (sl < d) val[u] = X_t[(size_t)sl * n + sample];
                            } else {
                                val[u] = (UPDATE || (INERTIA && sample_weight != nullptr)) ? sample_weight[sample] : TX(1);
                            }
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (at[u] < 0) continue;
                    if (pair[u]) {
                        queue[at[u]] = idx[u];
                        queue[at[u] + 1] = prv[u];
                    } else {
                        *reinterpret_cast<TX*>(queue + at[u]) = val[u];
                    }
                }
            }
        }
    }
    if (UPDATE) {
        // The moved samples: thread (entry, word) takes the term of feature `word` (word d: of the
        // weight) off the old cluster and adds it to the new one - the same fixed-point terms
        // a tile would have added.  Four items per thread and pass, their reads issued together.
        const int n_moved = (int)min(moved_count, (unsigned int)m_cap);
        const int wpe = d + 1, total = n_moved * wpe;
        constexpr int U = 4;
        for (int first = 0; first < total; first += U * THREADS) {
            TX xv[U], wv[U];
            uint32_t from_c[U], to_c[U];
            int word[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int item = first + u * THREADS + (int)threadIdx.x;
                word[u] = -1;
                xv[u] = TX(1);
                wv[u] = TX(0);
                from_c[u] = to_c[u] = 0u;
                if (item < total) {
                    const int e = item / wpe;
                    const uint32_t* entry = moved + e * SCR_MOVED_WORDS;
                    const uint32_t sample = entry[0];
                    if (sample != QUEUE_FREE) {
                        word[u] = item - e * wpe;
                        from_c[u] = entry[1];
                        to_c[u] = entry[2];
                        wv[u] = sample_weight[sample];
                        if (word[u] < d) xv[u] = X_t[(size_t)word[u] * n + sample];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (word[u] < 0) continue;
                const double magic = fix_magic(q_lds[word[u]]);
                // x * w is exact in fp64 (fp32 inputs); one rounding, to a multiple of 2^-q (the weight's word: w itself)
                const double v = word[u] < d ? fma((double)xv[u], (double)wv[u], magic) : (double)wv[u] + magic;
                const unsigned long long term = to_fixed_q(v, magic);
                const int slot = word[u] < d ? word[u] : d_even;
                atomicAdd(acc + to_c[u] * (uint32_t)acc_stride + slot, term);
                atomicSub(acc + from_c[u] * (uint32_t)acc_stride + slot, term);
            }
        }
    }
    __syncthreads();  // entries complete
    if constexpr (!F64) {
        const int n_queued = n_noted;
        double magic_lane = 0.0;  // lane f: of feature f; lane d: of the weights
        double magic_w64 = 0.0;   // d = 64 leaves no lane for the weights: lane 0 adds them as well
        if (UPDATE && n_queued > 0) {
            magic_lane = fix_magic(q_exp[lane < d ? lane : d]);
            if (d == 64) magic_w64 = fix_magic(q_exp[64]);
        }
        for (int e = wave; e < n_queued; e += WAVES) {
            const uint32_t* entry = queue + e * QW;
            const uint32_t sample = entry[Q_INDEX];
            if (sample == QUEUE_FREE) continue;  // reserved by a column that was redone instead
            const TX* xe = reinterpret_cast<const TX*>(entry);
            const int bc = evaluate_sample([&](const int f) __attribute__((always_inline)) { return xe[f]; });
            if (lane == 0) {
                labels[sample] = (uint32_t)bc;
                if (UPDATE) changed += entry[Q_PREV] != (uint32_t)bc ? 1u : 0u;
            }
            if constexpr (INERTIA) {
                float sq = 0.0f;
                if (lane < d) {
                    const float diff = (float)xe[lane] - ct[lane * kp + bc];
                    sq = diff * diff;
                }
                sq = kmx_wave_sum<float>(sq);
                if (lane == 0) inertia_lane += (double)(sq * (float)xe[NKF]);
            }
            if (UPDATE) {
                // lane f adds feature f, lane d the weight: the same fixed-point terms as above;
                // when the sums are only corrected, a sample that stays in its cluster adds
                // nothing and one that moves is taken off the old cluster
                const uint32_t prev = entry[Q_PREV];
                const double wq = (double)xe[NKF];  // (the weight follows the features)
                if (lane <= d && (full_mode || prev != (uint32_t)bc)) {
                    const double term = lane < d ? fma((double)xe[lane], wq, magic_lane) : wq + magic_lane;
                    const unsigned long long fixed = to_fixed_q(term, magic_lane);
                    const int word = lane < d ? lane : d_even;
                    atomicAdd(acc + bc * acc_stride + word, fixed);
                    if (!full_mode) atomicSub(acc + prev * (uint32_t)acc_stride + word, fixed);
                }
                if (d == 64 && lane == 0 && (full_mode || prev != (uint32_t)bc)) {
                    const unsigned long long fixed = to_fixed_q(wq + magic_w64, magic_w64);
                    atomicAdd(acc + bc * acc_stride + d_even, fixed);
                    if (!full_mode) atomicSub(acc + prev * (uint32_t)acc_stride + d_even, fixed);
                }
            }
        }
    } else {
        // fp64 inputs: sixteen noted samples at a time on the fp64 matrix cores
        // (v_mfma_f64_16x16x4_f64: A = 16 centroids x 4 features, lane l: centroid l % 16, feature
        // l / 16; B = 4 features x 16 samples, lane l: feature l / 16, sample l % 16; D: lane l holds
        // rows l / 16 + 4 r, r = 0..3, of column l % 16).  Lane (g, m) = (l / 16, l % 16) gathers
        // features 4 s + g of sample m straight from memory, all of them in flight together, and
        // afterwards adds the same values to the sums of the sample's cluster.
        typedef double v4d __attribute__((ext_vector_type(4)));
        constexpr int NS = 4 * NK;  // K steps of four features
        const int g4 = lane >> 4, m16 = lane & 15;
        const int n_groups = (n_noted + 15) >> 4;
        for (int gq = wave; gq < n_groups; gq += WAVES) {
            const int slot = 16 * gq + m16;
            const uint32_t sample = slot < n_noted ? qlist[slot] : QUEUE_FREE;
            const bool valid = sample != QUEUE_FREE;  // (free: reserved and never written)
            const size_t at = valid ? (size_t)sample : 0;
            double xk[NS];
#pragma unroll
            for (int s4 = 0; s4 < NS; ++s4) {
                const int f = 4 * s4 + g4;
                xk[s4] = f < d ? (double)X_t[(size_t)f * n + at] : 0.0;
            }
            const double wv = UPDATE ? (double)sample_weight[at] : 1.0;
            const uint32_t prev = UPDATE ? labels_prev[at] : 0u;
            double bs = -kmx_inf<double>();
            int bc = 0x7fffffff;
            for (int cb = 0; cb < (kp >> 4); ++cb) {
                const TX* hp = hxx + 16 * cb + g4;
                v4d a = {-(double)hp[0], -(double)hp[4], -(double)hp[8], -(double)hp[12]};
#pragma unroll
                for (int s4 = 0; s4 < NS; ++s4) {
                    const int f = 4 * s4 + g4;
                    const double af = f < d ? (double)ctx[f * kp + 16 * cb + m16] : 0.0;
                    a = __builtin_amdgcn_mfma_f64_16x16x4f64(af, xk[s4], a, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)  // increasing centroid index inside the lane; strict
                    if (a[r] > bs) {
                        bs = a[r];
                        bc = 16 * cb + g4 + 4 * r;
                    }
            }
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const double ob = __shfl_xor(bs, off, 64);
                const int oc = __shfl_xor(bc, off, 64);
                if (ob > bs || (ob == bs && oc < bc)) {
                    bs = ob;
                    bc = oc;
                }
            }
            if (bc == 0x7fffffff) bc = 0;  // no score compares: the reference's running arg-min keeps 0
            if (valid && g4 == 0) {
                labels[sample] = (uint32_t)bc;
                if (UPDATE) changed += prev != (uint32_t)bc ? 1u : 0u;
            }
            if (UPDATE && valid && (full_mode || prev != (uint32_t)bc)) {
                // the same fixed-point terms as a tile adds; when the sums are only corrected, a
                // sample that moves is taken off the old cluster
#pragma unroll
                for (int s4 = 0; s4 < NS; ++s4) {
                    const int f = 4 * s4 + g4;
                    if (f < d) {
                        const double magic = fix_magic(q_lds[f]);
                        const unsigned long long term = to_fixed_q(fma(xk[s4], wv, magic), magic);
                        atomicAdd(acc + bc * acc_stride + f, term);
                        if (!full_mode) atomicSub(acc + prev * (uint32_t)acc_stride + f, term);
                    }
                }
                if (g4 == 0) {
                    const double magic_w = fix_magic(q_lds[d]);
                    const unsigned long long term = to_fixed_q(wv + magic_w, magic_w);
                    atomicAdd(acc + bc * acc_stride + d_even, term);
                    if (!full_mode) atomicSub(acc + prev * (uint32_t)acc_stride + d_even, term);
                }
            }
        }
    }

    if (UPDATE && changed) atomicAdd(&changed_block, changed);
    if (lane == 0 && n_uncertain) atomicAdd(&uncertain_block, n_uncertain);
    if constexpr (INERTIA) {
        // wave totals in order, then the waves in order
        const double wsum = kmx_wave_sum<double>(inertia_lane);
        double* wave_tot = reinterpret_cast<double*>(wave_key);
        __syncthreads();
        if (lane == 0) wave_tot[wave] = wsum;
        __syncthreads();
        if (threadIdx.x == 0) {
            double total = 0.0;
            for (int w2 = 0; w2 < WAVES; ++w2) total += wave_tot[w2];
            inertia_partial[blockIdx.x] = total;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0 && uncertain_block && uncertain_count != nullptr)
        atomicAdd(uncertain_count, uncertain_block);
    if (UPDATE) {
        if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
        const int n_out = (d + 1) * k;  // gsum is feature-major, (d + 1, k), and has no spare row
        // every workgroup starts at another word: the workgroups finish together and would
        // otherwise queue up on the same addresses
        const int rot = (int)(((int64_t)blockIdx.x * n_out) / gridDim.x);
        for (int jy = threadIdx.x; jy < n_out; jy += THREADS) {
            const int jx = jy + rot < n_out ? jy + rot : jy + rot - n_out;
            const int f = jx / k, c = jx - f * k;
            const unsigned long long v = acc[c * acc_stride + (f < d ? f : d_even)];
            if (v) atomicAdd(gsum + jx, v);
        }
        // The workgroup that gets done last finishes the iteration (empty-cluster list, division,
        // shift, convergence test, what the next step needs) instead of a launch of its own, which
        // would cost its launch, its first round trips to memory and the gap between two dependent
        // launches.  What the workgroups hand over - sums, changed-label count, the counter of
        // samples evaluated in fp32 - went through device-scope atomics, performed at the memory
        // side; each workgroup waits for its own before it draws its ticket, and the last one
        // reads them with device-scope loads.  No device-wide fence.
        if (fuse_tail) {
            __shared__ unsigned int is_last;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0) is_last = (atomicAdd(&status->ticket, 1u) == gridDim.x - 1) ? 1u : 0u;
            __syncthreads();
            if (is_last != 0u) {
                // (the accumulators are flushed: their LDS holds the (d + 1) k sums as floats)
                lloyd_small_finalize_body<TX, true, true>(gsum, q_exp, tail, reinterpret_cast<TX*>(smem_raw));
                if (threadIdx.x == 0) status->ticket = 0u;
            }
        }
    }
}

// ---------------------------------------------------------------------------- diagnostics

__global__ void absmax_fill_zero(unsigned int* p) {
    if (threadIdx.x == 0) *p = 0u;
}

// max |X_t| over all features into *xmax_bits (zero on entry), one workgroup per 1024 values.
__global__ __launch_bounds__(256) void screen_absmax_kernel(const float* __restrict__ X_t,
                                                            unsigned int* __restrict__ xmax_bits,
                                                            int64_t count) {
    float m = 0.0f;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256)
        m = fmaxf(m, fabsf(X_t[i]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((threadIdx.x & 63) == 0) atomicMax(xmax_bits, __float_as_uint(m));
}

// The approximate scores exactly as lloyd_screen_kernel forms them (same scaling, same split,
// same MFMA sequence), written out with the error bound the kernel would use: one wave per 32
// samples.  scores (k, n) and half_norms (k) are in scaled units (x * scale, c * scale).
template <int NK>
__global__ __launch_bounds__(64) void screen_scores_kernel(
    const float* __restrict__ X_t, const float* __restrict__ centroids_t,
    const unsigned int* __restrict__ xmax_bits, float* __restrict__ scores,
    float* __restrict__ bounds, float* __restrict__ half_norms, float* __restrict__ scale_out,
    int64_t n, int d, int k) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int n_cb = (k + 31) >> 5;
    v8h* afh = reinterpret_cast<v8h*>(smem_raw);
    v8h* afl = afh + n_cb * NK * 64;
    float* hneg = reinterpret_cast<float*>(afl + n_cb * NK * 64);
    __shared__ unsigned int hmax_bits;
    const float xmax = __uint_as_float(*xmax_bits);
    // d <= 32: the arithmetic of lloyd_screen_kernel (its scale; -0.5||c||^2 in the spare feature
    // slot d when there is one); wider: that of the wide path's label kernel (data scaled into
    // [2^14, 2^15), -0.5||c||^2 as the accumulators' start)
    const bool narrow = d <= 32;
    const float xs = (xmax > 0.0f && xmax < kmx_inf<float>())
                         ? ldexpf(1.0f, (narrow ? SCR_SCALE_EXP - 1 : 14) - ilogbf(xmax))
                         : 1.0f;
    const bool hk = narrow && d % 16 != 0;
    const int spare = 16 * ((d + 15) / 16) - 1;  // the feature slot that then carries -0.5||c||^2
    if (threadIdx.x == 0) hmax_bits = 0;
    __syncthreads();
    for (int idx = threadIdx.x; idx < n_cb * NK * 64; idx += 64) {
        const int l = idx & 63, s = (idx >> 6) % NK, cb = (idx >> 6) / NK;
        const int c = 32 * cb + (l & 31);
        v8h hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = 16 * s + 2 * i + (l >> 5);
            float v = (c < k && f < d) ? centroids_t[(size_t)f * k + c] * xs : 0.0f;
            if (hk && f == spare) {
                v = -kmx_inf<float>();
                if (c < k) {
                    float sq = 0.0f;
                    for (int g = 0; g < d; ++g) {
                        const float cv = centroids_t[(size_t)g * k + c] * xs;
                        sq += cv * cv;
                    }
                    v = -(sq / 2.0f) * (1.0f / SCR_HK_X1);
                }
            }
            const _Float16 hb = (_Float16)v;
            hi[i] = hb;
            lo[i] = (_Float16)(v - (float)hb);
            if (hk && f == spare && !(c < k)) {
                hi[i] = (_Float16)0.0f;
                lo[i] = hb;
            }
        }
        afh[idx] = hi;
        afl[idx] = lo;
    }
    for (int idx = threadIdx.x; idx < n_cb * 32; idx += 64) {
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
            atomicMax(&hmax_bits, __float_as_uint(sq / 2.0f));
            if (blockIdx.x == 0) half_norms[c] = sq / 2.0f;
        }
        hneg[idx] = v;
    }
    __syncthreads();
    const int lane = threadIdx.x, h = lane >> 5, j = lane & 31;
    const int64_t i0 = (int64_t)blockIdx.x * 32 + j;
    const float hmax = __uint_as_float(hmax_bits);
    const float cmax = sqrtf(2.0f * hmax), abs_term = SCR_ERR_ABS * sqrtf((float)d);
    const float round_term = SCR_ERR_ROUND * 51.0f * (float)((d + 15) / 16);
    v8h xh[NK], xl[NK];
    float ss = 0.0f;
#pragma unroll
    for (int s = 0; s < NK; ++s)
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const int f = 16 * s + 2 * i + h;
            const float x0 = (f < d && i0 < n) ? X_t[(size_t)f * n + i0] : 0.0f;
            const float x1 = (f + 2 < d && i0 < n) ? X_t[(size_t)(f + 2) * n + i0] : 0.0f;
            v2f p = {x0 * xs, x1 * xs};
            if (hk && f == spare) p[0] = SCR_HK_X1;
            if (hk && f + 2 == spare) p[1] = SCR_HK_X1;
            const v2h hh = __builtin_convertvector(p, v2h);
            const v2f r = p - __builtin_convertvector(hh, v2f);
            const v2h ll = __builtin_convertvector(r, v2h);
            xh[s][i] = hh[0];
            xh[s][i + 1] = hh[1];
            xl[s][i] = ll[0];
            xl[s][i + 1] = ll[1];
            if (f < d) ss = fmaf(p[0], p[0], ss);
            if (f + 2 < d) ss = fmaf(p[1], p[1], ss);
        }
    const float nrm = ss + __shfl_xor(ss, 32, 64);
    if (h == 0 && i0 < n)
        bounds[i0] = fmaf((SCR_ERR_SPLIT + round_term) * cmax + abs_term, __builtin_amdgcn_sqrtf(nrm),
                          round_term * hmax + abs_term * cmax +
                              (hk ? SCR_ERR_HNEG * hmax + SCR_ERR_ABS * SCR_HK_X1 : 0.0f));
    if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = xs;
    for (int cb = 0; cb < n_cb; ++cb) {
        const float4* hp = reinterpret_cast<const float4*>(hneg + cb * 32 + h * 16);
        v16f a;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 v4 = hp[q];
            a[4 * q] = hk ? 0.0f : v4.x;
            a[4 * q + 1] = hk ? 0.0f : v4.y;
            a[4 * q + 2] = hk ? 0.0f : v4.z;
            a[4 * q + 3] = hk ? 0.0f : v4.w;
        }
#pragma unroll
        for (int s = 0; s < NK; ++s) {
            const v8h ah = afh[(cb * NK + s) * 64 + lane];
            const v8h al = afl[(cb * NK + s) * 64 + lane];
            a = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xh[s], a, 0, 0, 0);
            a = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, xl[s], a, 0, 0, 0);
            a = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, xh[s], a, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int c = 32 * cb + 8 * (r >> 2) + 4 * h + (r & 3);
            if (c < k && i0 < n) scores[(size_t)c * n + i0] = a[r];
        }
    }
}

}  // namespace

// K steps the kernel runs with: as many as the features need - or three for 17 to 32 features
// whose accumulators and operands do not fit the half of a compute unit's LDS that a workgroup
// of the two-step kernel gets: the three-step kernel is one workgroup with all of it (its third
// step then holds no feature: zero operands, exact), which keeps such shapes off the wide path.
static int screen_k_steps(int d, int k, bool update, int esize = 4) {
    const int nk = (d + 15) / 16;
    if (nk == 2 && screen_lds(d, k, 2, update, esize).off_queue > scr_lds_max(2) &&
        screen_lds(d, k, 3, update, esize).off_queue <= scr_lds_max(3))
        return 3;
    return nk;
}

// Shapes the screened step covers: d <= 64 (one to four K steps of 16 features), everything within the workgroup's LDS, byte offsets
// inside two rows of X_t within 32 bits.
bool kmx_mfma_screen_fits(int64_t n, int d, int k) {
    if (d < 1 || d > 64 || k < 16 || n >= ((int64_t)1 << 29)) return false;
    const int nk = screen_k_steps(d, k, true);
    return screen_lds(d, k, nk, true).off_queue <= scr_lds_max(nk);
}

// The same step on fp64 inputs: the centroids in LDS are fp64, and the list of noted samples
// takes the place of the queue.
static bool screen_fits_f64(int64_t n, int d, int k) {
    if (d < 1 || d > 64 || k < 16 || n >= ((int64_t)1 << 29)) return false;
    const int nk = screen_k_steps(d, k, true, 8);
    return screen_lds(d, k, nk, true, 8).off_queue <= scr_lds_max(nk);
}

// Left to the library it is used wherever it fits (measured at 2e6 x 32, 64 clusters: 2.0x the
// fp64 matrix-core step); KMX_FLAG_LABELS_F32 - "no fp16 screen" - switches it off.
bool kmx_mfma_screen_f64_supported(int64_t n, int d, int k, uint32_t flags) {
    if ((flags & KMX_FLAG_LABELS_MASK) == KMX_FLAG_LABELS_F32) return false;
    return screen_fits_f64(n, d, k);
}

// The labels-only kernel needs no accumulators: shapes whose fused step does not fit the LDS
// can still have their labels screened (the sums are then taken per bucket of samples).
bool kmx_mfma_screen_labels_fits(int64_t n, int d, int k) {
    if (d < 1 || d > 64 || k < 16 || n >= ((int64_t)1 << 29)) return false;
    const int nk = screen_k_steps(d, k, false);
    return screen_lds(d, k, nk, false).off_queue <= scr_lds_max(nk);
}

// Left to the library it is chosen where it is the faster one: the all-fp32 step pays d / 2 fp32
// MFMAs per block of 32 centroids, the screen three fp16 ones plus the split and the certificate
// whatever d is; measured on 2e6 samples the screen wins from d = 10 on, from d = 8 for k >= 64
// and from d = 6 for k >= 128 (at d = 2 it is 30 % slower, at d = 16, k = 128 36 % faster).
// KMX_FLAG_LABELS_F32 switches it off (all-fp32 scores on the matrix cores, lloyd_mfma.hip),
// KMX_FLAG_LABELS_SCREEN selects it wherever it is possible.
bool kmx_mfma_screen_supported(int64_t n, int d, int k, uint32_t flags) {
    if ((flags & KMX_FLAG_LABELS_MASK) == KMX_FLAG_LABELS_F32) return false;
    if (!kmx_mfma_screen_fits(n, d, k)) return false;
    if ((flags & KMX_FLAG_LABELS_MASK) == KMX_FLAG_LABELS_SCREEN) return true;
    return d >= 10 || (d >= 8 && k >= 64) || (d >= 6 && k >= 128);
}

namespace {
template <bool UPDATE, bool INERTIA = false, typename TX = float>
int32_t launch_screen(const void* X_t, const void* w, const void* centroids_t, const uint32_t* labels_prev,
                      uint32_t* labels, kmx_lloyd_status* status, const unsigned int* absmax,
                      const int* q_exp, unsigned long long* gsum, uint32_t* uncertain_count,
                      const float* norms, int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream,
                      double* inertia_partial = nullptr, int* grid_out = nullptr,
                      const LloydTail<TX>* tail = nullptr) {
    constexpr int ES = (int)sizeof(TX);
    static_assert(ES == 4 || !INERTIA, "fp64 inputs: labels and inertia are two calls");
    if (!(ES == 8 ? screen_fits_f64(n, d, k)
                  : (UPDATE ? kmx_mfma_screen_fits(n, d, k) : kmx_mfma_screen_labels_fits(n, d, k))))
        return KMX_ERR_UNSUPPORTED;
    const int nk = screen_k_steps(d, k, UPDATE, ES);
    const int waves = scr_waves(nk);
    const int64_t n_wtiles = kmx_cdiv(n, 64);
    int64_t grid = kmx_cdiv(n_wtiles, waves);
    const int per_cu = waves >= 8 ? 1 : 2;
    const int cap = (wgs_per_cu > 0 ? wgs_per_cu : per_cu) * kmx_num_cus();
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
    auto aligned16 = [](const void* p) { return (((uintptr_t)p) & 15) == 0; };
    // (the fast path addresses a lane's rows with 32-bit byte offsets from the tile's address in row 0)
    const int vec_ok = ((uint64_t)d * (uint64_t)n * (uint64_t)ES < ((uint64_t)1 << 32)) && (n % 4 == 0) && aligned16(X_t) &&
                       aligned16(labels) && aligned16(w) &&
                       aligned16(labels_prev);
    const size_t lds = screen_lds(d, k, nk, UPDATE, ES).total;
    // -0.5||c||^2 in a spare feature slot of the last K step whenever there is one
    const bool hk = d % 16 != 0;
#define KMX_SCR_LAUNCH(NK_, HK_)                                                                            \
    do {                                                                                                    \
        if (lds > 64 * 1024) {                                                                              \
            const hipError_t e = hipFuncSetAttribute(                                                       \
                reinterpret_cast<const void*>(&lloyd_screen_kernel<TX, NK_, UPDATE, HK_, INERTIA>),         \
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                      \
            if (e != hipSuccess) return (int32_t)e;                                                         \
        }                                                                                                   \
        hipLaunchKernelGGL((lloyd_screen_kernel<TX, NK_, UPDATE, HK_, INERTIA>), dim3((unsigned)grid),      \
                           dim3(64 * scr_waves(NK_)), lds, stream, (const TX*)X_t, (const TX*)w,            \
                           (const TX*)centroids_t, labels_prev, labels, status, absmax, q_exp, gsum,        \
                           uncertain_count, norms, n, d, k, vec_ok, inertia_partial,                        \
                           tail ? *tail : LloydTail<TX>(), tail ? 1 : 0);                                   \
    } while (0)
    if (nk == 1) {
        if (hk) KMX_SCR_LAUNCH(1, true); else KMX_SCR_LAUNCH(1, false);
    } else if (nk == 2) {
        if (hk) KMX_SCR_LAUNCH(2, true); else KMX_SCR_LAUNCH(2, false);
    } else if (nk == 3) {
        if (hk) KMX_SCR_LAUNCH(3, true); else KMX_SCR_LAUNCH(3, false);
    } else {
        if (hk) KMX_SCR_LAUNCH(4, true); else KMX_SCR_LAUNCH(4, false);
    }
#undef KMX_SCR_LAUNCH
    KMX_LAUNCH_CHECK();
    if (grid_out) *grid_out = (int)grid;
    return KMX_OK;
}
}  // namespace

// Screened fused step.  `uncertain_count`: one word the kernel adds the number of samples it
// evaluated in fp32 to (zero on entry; the finalisation that follows moves it to the next word
// and clears it).  `absmax`: bits of max|X_t row| per feature, as kmx_lloyd_mfma_prepare leaves
// them; `norms`: ||x_i|| per sample (kmx_sample_norms).
// `tail` (may be null): what the finalisation of the iteration needs; the workgroup of the step
// that gets done last then runs it, and no finalisation launch must follow.
int32_t kmx_lloyd_step_mfma_screen(const void* X_t, const void* w, const void* centroids_t,
                                   const uint32_t* labels_prev, uint32_t* labels,
                                   kmx_lloyd_status* status, const unsigned int* absmax,
                                   const int* q_exp, unsigned long long* gsum,
                                   uint32_t* uncertain_count, const float* norms, int64_t n, int d,
                                   int k, int wgs_per_cu, hipStream_t stream, const LloydTail<float>* tail) {
    return launch_screen<true>(X_t, w, centroids_t, labels_prev, labels, status, absmax, q_exp, gsum,
                               uncertain_count, norms, n, d, k, wgs_per_cu, stream, nullptr, nullptr, tail);
}

// The same on fp64 inputs (X_t, w, centroids_t and the tail's arrays are fp64; norms stay fp32).
int32_t kmx_lloyd_step_mfma_screen_f64(const void* X_t, const void* w, const void* centroids_t,
                                       const uint32_t* labels_prev, uint32_t* labels,
                                       kmx_lloyd_status* status, const unsigned int* absmax,
                                       const int* q_exp, unsigned long long* gsum,
                                       uint32_t* uncertain_count, const float* norms, int64_t n, int d,
                                       int k, int wgs_per_cu, hipStream_t stream, const LloydTail<double>* tail) {
    return launch_screen<true, false, double>(X_t, w, centroids_t, labels_prev, labels, status, absmax, q_exp, gsum,
                                              uncertain_count, norms, n, d, k, wgs_per_cu, stream, nullptr, nullptr,
                                              tail);
}

// Labels only, screened the same way: nothing but X and the centroids is needed (the scale comes
// from the centroids, each tile takes the norms of its samples itself).
int32_t kmx_assign_labels_mfma_screen(const void* X_t, const void* centroids_t, uint32_t* labels,
                                      int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream) {
    return launch_screen<false>(X_t, nullptr, centroids_t, nullptr, labels, nullptr, nullptr, nullptr,
                                nullptr, nullptr, nullptr, n, d, k, wgs_per_cu, stream);
}

// Labels only on fp64 inputs (the shapes of the fused fp64 step).
int32_t kmx_assign_labels_mfma_screen_f64(const void* X_t, const void* centroids_t, uint32_t* labels,
                                          int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream) {
    return launch_screen<false, false, double>(X_t, nullptr, centroids_t, nullptr, labels, nullptr, nullptr, nullptr,
                                               nullptr, nullptr, nullptr, n, d, k, wgs_per_cu, stream);
}

// The same inside the iteration loop (no work once the run's state is terminal).
int32_t kmx_lloyd_labels_mfma_screen(const void* X_t, const void* centroids_t, uint32_t* labels,
                                     kmx_lloyd_status* status, int64_t n, int d, int k, int wgs_per_cu,
                                     hipStream_t stream) {
    return launch_screen<false>(X_t, nullptr, centroids_t, nullptr, labels, status, nullptr, nullptr, nullptr,
                                nullptr, nullptr, n, d, k, wgs_per_cu, stream);
}

// The same with the weighted inertia of the labelling summed on the way: one fp64 partial sum per
// workgroup in inertia_partial (room for 8 per compute unit), *n_partials receives how many.
int32_t kmx_assign_labels_inertia_mfma_screen(const void* X_t, const void* w, const void* centroids_t,
                                              uint32_t* labels, double* inertia_partial, int* n_partials,
                                              int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream) {
    return launch_screen<false, true>(X_t, w, centroids_t, nullptr, labels, nullptr, nullptr, nullptr, nullptr,
                                      nullptr, nullptr, n, d, k, wgs_per_cu, stream, inertia_partial, n_partials);
}

// Diagnostics of the screen: approximate scores and error bounds as the fused step forms them.
int32_t kmx_screen_scores_impl(const float* X_t, const float* centroids_t, float* scores,
                               float* bounds, float* half_norms, float* scale, unsigned int* scratch,
                               int64_t n, int d, int k, hipStream_t stream) {
    if (d < 1 || d > 256 || k < 1 || n >= ((int64_t)1 << 29)) return KMX_ERR_UNSUPPORTED;
    const int nk16 = (d + 15) / 16;
    const int nk = nk16 <= 1 ? 1 : nk16 <= 2 ? 2 : nk16 <= 4 ? 4 : nk16 <= 8 ? 8 : 16;
    const int n_cb = (k + 31) / 32;
    const size_t lds = (size_t)n_cb * nk * 64 * 32 + (size_t)n_cb * 32 * 4;
    if (lds > 64 * 1024) return KMX_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(absmax_fill_zero, dim3(1), dim3(64), 0, stream, scratch);
    hipLaunchKernelGGL(screen_absmax_kernel, dim3(256), dim3(256), 0, stream, X_t, scratch, (int64_t)d * n);
    const unsigned grid = (unsigned)kmx_cdiv(n, 32);
#define KMX_DIAG_CASE(NK)                                                                               \
    hipLaunchKernelGGL((screen_scores_kernel<NK>), dim3(grid), dim3(64), lds, stream, X_t, centroids_t, \
                       scratch, scores, bounds, half_norms, scale, n, d, k)
    switch (nk) {
        case 1: KMX_DIAG_CASE(1); break;
        case 2: KMX_DIAG_CASE(2); break;
        case 4: KMX_DIAG_CASE(4); break;
        case 8: KMX_DIAG_CASE(8); break;
        default: KMX_DIAG_CASE(16); break;
    }
#undef KMX_DIAG_CASE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

namespace {
// ||x_i|| in fp32, features in order; one thread per sample (consecutive threads, consecutive
// addresses in every feature row).
// (fp64 inputs: rounded to fp32 first, as the screen sees them)
template <typename TX>
__global__ __launch_bounds__(256) void sample_norms_kernel(const TX* __restrict__ X_t,
                                                           float* __restrict__ norms, int64_t n, int d) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float sq = 0.0f;
#pragma unroll 8
    for (int f = 0; f < d; ++f) {
        const float v = (float)X_t[(size_t)f * n + i];
        sq = fmaf(v, v, sq);
    }
    norms[i] = sqrtf(sq);
}
}  // namespace

int32_t kmx_sample_norms(const void* X_t, float* norms, int64_t n, int d, int dtype, hipStream_t stream) {
    const dim3 grid((unsigned)kmx_cdiv(n, 256));
    if (dtype == KMX_F64)
        hipLaunchKernelGGL(sample_norms_kernel<double>, grid, dim3(256), 0, stream, (const double*)X_t, norms, n, d);
    else
        hipLaunchKernelGGL(sample_norms_kernel<float>, grid, dim3(256), 0, stream, (const float*)X_t, norms, n, d);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
