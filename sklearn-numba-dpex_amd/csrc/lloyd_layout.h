// Workspace layout and kernel selection of the Lloyd iteration, shared by the vector-ALU
// and MFMA implementations.
#pragma once

#include "kmx_common.h"
#include "lloyd_tail.h"

constexpr int KMX_VARIANT_STREAM = 0;    // wide samples: features re-read per centroid window
constexpr int KMX_VARIANT_REGISTER = 1;  // samples held in registers, centroids in SGPRs
constexpr int KMX_VARIANT_MFMA = 3;      // fp32 distances on the matrix cores, LDS accumulators
constexpr int KMX_VARIANT_MFMA_WIDE = 4; // fp32 matrix cores, samples in registers, global sums
constexpr int KMX_VARIANT_MFMA_F64 = 5;  // fp64 distances on the matrix cores, LDS accumulators
constexpr int KMX_VARIANT_GEMM = 6;      // labels by a tiled matrix-core product (any shape), bucketed sums
constexpr int KMX_VARIANT_FEWK = 8;      // fp32, up to 16 clusters, 65 .. 1792 features: a tile of samples in LDS serves labels and sums

constexpr int KMX_ACC_LDS = 1;
constexpr int KMX_ACC_GLOBAL = 2;
constexpr int KMX_ACC_BUCKET = 3;  // labels-only kernel, then sums per bucket of samples (lloyd_bucket.hip)

constexpr int KMX_MAX_PARTIALS = 1024;          // upper bound on fused-step workgroups
constexpr size_t KMX_LDS_ACC_LIMIT = 40000;     // bytes of (fp64) LDS accumulators per workgroup
constexpr size_t KMX_GLOBAL_COPIES_BYTES = 64u << 20;

// Kernel selection comes from the caller's `flags` (KMX_FLAG_* of the public header) and from
// nothing else: the library reads no environment variable and keeps no selection state.
// Forced path (KMX_VARIANT_* or -1), workgroups per compute unit (0 = the kernel's default)
// and sample columns per lane of the matrix-core kernels (0 = default) out of the flags:
static inline int kmx_flags_forced_variant(uint32_t flags) {
    switch (flags & KMX_FLAG_PATH_MASK) {
        case KMX_FLAG_PATH_STREAM: return 0;
        case KMX_FLAG_PATH_REGISTER: return 1;
        case KMX_FLAG_PATH_MFMA: return 3;
        case KMX_FLAG_PATH_GEMM: return 6;
        default: return -1;
    }
}
static inline int kmx_flags_wgs_per_cu(uint32_t flags) {
    const int x = (int)((flags >> 8) & 0xfu);
    return (x >= 1 && x <= 8) ? x : 0;
}
static inline int kmx_flags_cols(uint32_t flags) {
    const int x = (int)((flags >> 12) & 0x7u);
    return (x == 2 || x == 4) ? x : 0;
}
static inline bool kmx_flags_valid(uint32_t flags) {
    if (flags & ~(uint32_t)0x7f3f) return false;
    if ((flags & KMX_FLAG_PATH_MASK) > KMX_FLAG_PATH_GEMM) return false;
    if ((flags & KMX_FLAG_LABELS_MASK) == KMX_FLAG_LABELS_MASK) return false;
    const uint32_t w = (flags >> 8) & 0xfu, c = (flags >> 12) & 0x7u;
    return w <= 8 && (c == 0 || c == 2 || c == 4);
}
// Shapes the fp32 matrix-core fused step covers (operands and accumulators fit in LDS), and
// those its wide-sample variant covers (samples in registers, centroids streamed).
bool kmx_mfma_supported(int d, int k);
bool kmx_mfma_wide_supported(int d, int k);
bool kmx_mfma_f64_supported(int d, int k);
bool kmx_mfma_f64_labels_supported(int d, int k);  // without the accumulators in LDS
// labels of any shape by a tiled matrix-core product (lloyd_gemm.hip)
int32_t kmx_lloyd_gemm_labels(const void* X_t, const void* centroids_t, const void* half_norms,
                              uint32_t* labels, const kmx_lloyd_status* status, int64_t n, int d, int k,
                              int32_t dtype, hipStream_t stream);
int32_t kmx_lloyd_gemm_labels_listed(const void* X_t, const void* centroids_t, const void* half_norms,
                                     uint32_t* labels, const kmx_lloyd_status* status, const int* list,
                                     const unsigned int* list_count, int64_t n, int d, int k,
                                     hipStream_t stream);
// the same product screened on the fp16 matrix cores (lloyd_gemm_screen.hip), fp32 only
size_t kmx_gemm_screen_bytes(int64_t n);
bool kmx_gemm_screen_enabled(int64_t n, int d, int k, uint32_t flags);
const uint32_t* kmx_gemm_screen_counter(const char* area);
int32_t kmx_lloyd_gemm_screen_labels(const void* X_t, const void* centroids_t, const void* half_norms,
                                     const unsigned int* absmax, char* area, uint32_t* labels,
                                     const kmx_lloyd_status* status, int64_t n, int d, int k,
                                     hipStream_t stream);
// bucketed sums (lloyd_bucket.hip)
size_t kmx_bucket_bytes(int64_t n, int k);
int32_t kmx_bucket_order(const uint32_t* labels, const int* counts, int* offsets, const int* ranks,
                         int* order, int64_t n, int k, hipStream_t stream);
int32_t kmx_lloyd_bucket_sums(const void* X_t, const void* X_rowmajor, const void* w,
                              const uint32_t* labels_prev, const uint32_t* labels, void* sums,
                              kmx_lloyd_status* status, char* bucket, int64_t n, int d, int k,
                              int32_t dtype, hipStream_t stream);
// fp32 sums straight from the labels, accumulators of every cluster in LDS (lloyd_bucket.hip)
bool kmx_direct_sums_fits(int d, int k);
int32_t kmx_lloyd_direct_sums(const void* X_t, const void* w, const uint32_t* labels_prev,
                              const uint32_t* labels, const int* q_exp, unsigned long long* gsum,
                              kmx_lloyd_status* status, int64_t n, int d, int k, hipStream_t stream);
// fp32 matrix-core step with fp16 screening of the labels (lloyd_mfma_screen.hip): whether the
// shape fits the kernel at all, and whether the flags (or, left to the library, the measured
// break-even) select it
bool kmx_mfma_screen_fits(int64_t n, int d, int k);
bool kmx_mfma_screen_supported(int64_t n, int d, int k, uint32_t flags);
bool kmx_mfma_screen_f64_supported(int64_t n, int d, int k, uint32_t flags);  // fp64 inputs
// the same kernel without the sums (labels only): needs less LDS
bool kmx_mfma_screen_labels_fits(int64_t n, int d, int k);
// few clusters on wide samples, X read once (lloyd_fewk.hip)
bool kmx_fewk_supported(int d, int k);
int kmx_fewk_grid(int64_t n, int d, int k, int wgs_per_cu);
size_t kmx_fewk_partial_bytes(int d, int k);
int32_t kmx_lloyd_labels_mfma_screen(const void* X_t, const void* centroids_t, uint32_t* labels,
                                     kmx_lloyd_status* status, int64_t n, int d, int k, int wgs_per_cu,
                                     hipStream_t stream);
// screened label step of the wide path (lloyd_mfma_wide_screen.hip)
size_t kmx_wide_screen_bytes(int64_t n, int d, int k);
const int* kmx_wide_screen_list(const char* area, int d, int k);
bool kmx_wide_screen_enabled(int64_t n, int d, int k, uint32_t flags);
const uint32_t* kmx_wide_screen_counter(const char* area);

struct LloydLayout {
    int dpad;            // features per packed centroid row (multiple of 4, zero padded)
    int variant;         // KMX_VARIANT_*
    int acc_mode;        // KMX_ACC_*
    int n_partials;      // slots in `partial` (workgroups for LDS mode, copies for global mode)
    int k_for_gsum;      // n_clusters (size of the fixed-point sum array is (d + 1) * k)
    bool screen;         // KMX_VARIANT_MFMA with fp16-screened labels (variant code 61)
    bool screen64;       // fp64 inputs: the same screened fused step (variant code 71)
    bool gemm_screen;    // KMX_VARIANT_GEMM (fp32) with fp16-screened labels
    bool screen_labels;  // KMX_VARIANT_GEMM (fp32, d <= 64): labels by the screened kernel of variant 61 without its sums
    bool direct_sums;    // with screen_labels: sums straight from the labels (fixed point in LDS) instead of per bucket
    uint32_t flags;      // the caller's KMX_FLAG_* selection
    int wgs_per_cu;      // workgroups per compute unit asked for (0: the kernel's default)
    int cols;            // sample columns per lane asked for (0: the kernel's default)
    size_t off_status, off_scales, off_gsum, off_cpack, off_half, off_shift, off_bucket, off_wscreen, off_partial;
    size_t partial_bytes;
    size_t total;
    // Workgroups of the fused step: a few per compute unit (default 4), never more than the
    // partial slots.
    int grid_cap(int cus) const {
        const int g = (wgs_per_cu > 0 ? wgs_per_cu : 4) * cus;
        return g < partial_slots() ? g : partial_slots();
    }
    // Workgroups that may write partial sums (the labels-only kernel of the bucketed mode
    // writes none).
    int partial_slots() const { return acc_mode == KMX_ACC_BUCKET ? KMX_MAX_PARTIALS : n_partials; }
};

static inline int lloyd_reg_samples_per_thread(int d, int dtype) {
    if (dtype == KMX_F32) return d <= 16 ? 4 : (d <= 32 ? 2 : 1);
    return d <= 16 ? 2 : 1;
}


static inline LloydLayout lloyd_layout(int64_t n, int d, int k, int dtype, uint32_t flags) {
    LloydLayout L;
    L.flags = flags;
    L.wgs_per_cu = kmx_flags_wgs_per_cu(flags);
    L.cols = kmx_flags_cols(flags);
    const size_t s = kmx_dtype_size(dtype);
    L.dpad = (d + 3) & ~3;
    L.k_for_gsum = k;
    const size_t items = (size_t)(d + 1) * k;
    // (measured: fp32 rows beyond 64 features are no faster from registers than streamed twice)
    const bool reg_ok = d <= 64;
    L.variant = reg_ok ? KMX_VARIANT_REGISTER : KMX_VARIANT_STREAM;
    const int forced = kmx_flags_forced_variant(flags);
    const bool screen_labels_ok = dtype == KMX_F32 && n <= INT32_MAX &&
                                  (flags & KMX_FLAG_LABELS_MASK) != KMX_FLAG_LABELS_F32 &&
                                  kmx_mfma_screen_labels_fits(n, d, k);
    if (forced == KMX_VARIANT_STREAM) L.variant = KMX_VARIANT_STREAM;
    if (forced == KMX_VARIANT_REGISTER && reg_ok) L.variant = KMX_VARIANT_REGISTER;
    if (items * sizeof(double) <= KMX_LDS_ACC_LIMIT) {
        L.acc_mode = KMX_ACC_LDS;
        L.n_partials = KMX_MAX_PARTIALS;
    } else {
        L.acc_mode = KMX_ACC_GLOBAL;
        size_t copies = KMX_GLOBAL_COPIES_BYTES / (items * s);
        if (copies < 1) copies = 1;
        if (copies > 32) copies = 32;
        L.n_partials = (int)copies;
    }
    // (the screened step has the whole LDS of a compute unit and covers shapes the all-fp32
    // step, which stays within 64 KB, does not)
    // (their accumulators are 64-bit fixed point with a bound of their own)
    if (dtype == KMX_F32 && items * sizeof(float) <= KMX_LDS_ACC_LIMIT &&
        (kmx_mfma_supported(d, k) || kmx_mfma_screen_supported(n, d, k, flags)) &&
        (forced < 0 || forced == KMX_VARIANT_MFMA)) {
        L.variant = KMX_VARIANT_MFMA;
        L.acc_mode = KMX_ACC_LDS;
        L.n_partials = KMX_MAX_PARTIALS;
    }
    // (the wide path is built for many clusters: up to 256 the tiled product below is faster; and
    // up to 64 features the labels-only form of the screened kernel above, where its operands fit
    // the LDS, with sums per bucket of samples, is faster than either)
    // (its sample order, ranks and counts are 32-bit: kmx_lloyd_step_mfma_wide_f32 refuses more samples)
    else if (dtype == KMX_F32 && kmx_mfma_wide_supported(d, k) && n <= INT32_MAX &&
             ((forced < 0 && k > 256 && !screen_labels_ok) || forced == KMX_VARIANT_MFMA)) {
        L.variant = KMX_VARIANT_MFMA_WIDE;
        L.acc_mode = KMX_ACC_GLOBAL;  // always the global fixed-point sums (variant code 42)
    }
    else if (dtype == KMX_F64 && kmx_mfma_f64_supported(d, k) && (forced < 0 || forced == KMX_VARIANT_MFMA)) {
        L.variant = KMX_VARIANT_MFMA_F64;
        if (L.acc_mode != KMX_ACC_LDS) {
            // accumulators beyond what the vector-ALU kernels keep in LDS: one workgroup per
            // compute unit with all of its LDS, and only as many partial slots as that needs
            L.acc_mode = KMX_ACC_LDS;
            const int slots = 256 * (L.wgs_per_cu > 0 ? L.wgs_per_cu : 1);
            L.n_partials = slots < KMX_MAX_PARTIALS ? slots : KMX_MAX_PARTIALS;
        }
    }
    // (few clusters on wide samples: one read of X instead of two, or of a sort by label)
    else if (dtype == KMX_F32 && forced < 0 && kmx_fewk_supported(d, k)) {
        L.variant = KMX_VARIANT_FEWK;
        L.acc_mode = KMX_ACC_LDS;  // (per-workgroup sums, here kept in registers, then the fixed-point sums of the run)
        L.n_partials = 1;
    }
    const bool specialised = L.variant == KMX_VARIANT_MFMA || L.variant == KMX_VARIANT_MFMA_WIDE ||
                             L.variant == KMX_VARIANT_MFMA_F64 || L.variant == KMX_VARIANT_FEWK;
    if (n <= INT32_MAX && (!specialised || forced == KMX_VARIANT_GEMM)) {
        // No specialised fused kernel.  Beyond 16 clusters (one window of the streaming kernel; the
        // measured break-even lies between 16 and 32), or whenever the accumulators do not
        // fit in LDS (float atomics on global copies of the sums are slow on this hardware):
        // labels only, on the matrix cores -- the fp64 kernel when the centroid operands alone
        // fit in LDS, else the tiled product -- then bucketed sums.  Up to 16 clusters with
        // accumulators in LDS: the fused vector-ALU kernels.
        const bool matrix_ok = forced < 0 || forced == KMX_VARIANT_MFMA || forced == KMX_VARIANT_GEMM;
        // (fp64 beyond 64 features: the streaming kernel reads X twice with a thread per two
        // samples walking every feature; below a million samples the tiled product + bucketed
        // sums take 1.0 to 4 times less - 20 000 x 400, k = 10: 0.38 -> 0.09 ms -, above it
        // 10 to 20 % more)
        const bool stream_short_f64 = forced < 0 && dtype == KMX_F64 && L.variant == KMX_VARIANT_STREAM && n < 1000000;
        if (forced == KMX_VARIANT_GEMM) {
            L.variant = KMX_VARIANT_GEMM;
            L.acc_mode = KMX_ACC_BUCKET;
        } else if (matrix_ok && (k > 16 || L.acc_mode == KMX_ACC_GLOBAL || stream_short_f64)) {
            L.variant = (dtype == KMX_F64 && kmx_mfma_f64_labels_supported(d, k)) ? KMX_VARIANT_MFMA_F64
                                                                                 : KMX_VARIANT_GEMM;
            L.acc_mode = KMX_ACC_BUCKET;
        } else if (L.acc_mode == KMX_ACC_GLOBAL) {
            L.acc_mode = KMX_ACC_BUCKET;  // the vector-ALU kernel asked for, labels only
        }
        if (L.acc_mode == KMX_ACC_BUCKET) L.n_partials = 1;
    }
    L.screen = L.variant == KMX_VARIANT_MFMA && kmx_mfma_screen_supported(n, d, k, flags);
    // (where the fp64 matrix-core step would run with its accumulators in LDS)
    L.screen64 = dtype == KMX_F64 && L.variant == KMX_VARIANT_MFMA_F64 && L.acc_mode == KMX_ACC_LDS &&
                 kmx_mfma_screen_f64_supported(n, d, k, flags);
    L.gemm_screen = L.variant == KMX_VARIANT_GEMM && dtype == KMX_F32 && kmx_gemm_screen_enabled(n, d, k, flags);
    L.screen_labels = L.variant == KMX_VARIANT_GEMM && screen_labels_ok && !L.gemm_screen && forced != KMX_VARIANT_GEMM;
    L.direct_sums = L.screen_labels && kmx_direct_sums_fits(d, k);
    L.off_status = 0;
    // fixed-point scales of the matrix-core path: LloydScales, then (d + 1) * k int64 sums
    L.off_scales = kmx_align256(sizeof(kmx_lloyd_status));
    L.off_gsum = L.off_scales + kmx_align256(sizeof(float) * 2 * (size_t)(d + 1) + 64);
    L.off_cpack = L.off_gsum + kmx_align256(items * sizeof(long long));
    L.off_half = L.off_cpack + kmx_align256((size_t)k * L.dpad * s);
    L.off_shift = L.off_half + kmx_align256((size_t)k * s);
    L.off_bucket = L.off_shift + kmx_align256((size_t)kmx_cdiv(k, 4) * sizeof(double));  // one per finalisation workgroup (4 to 32 clusters each)
    // wide matrix-core path: counts (k), offsets (k + 1), sample order (n) and ranks inside the
    // cluster (n) as int32
    // screened path: the counter of samples evaluated in fp32 and its copy for the host (256
    // bytes), then ||x_i|| per sample
    const size_t bucket_bytes =
        (L.variant == KMX_VARIANT_MFMA_WIDE || L.acc_mode == KMX_ACC_BUCKET)
            ? ((size_t)2 * k + 1 + 2 * (size_t)n) * sizeof(int)
        : (L.screen || L.screen64) ? (size_t)256 + (size_t)n * sizeof(float)
                                           : 0;
    // wide matrix-core path: header, scaled half norms and fp16 parts of the centroids for the
    // screened label step (lloyd_mfma_wide_screen.hip)
    L.off_wscreen = L.off_bucket + kmx_align256(bucket_bytes);
    // (reserved whatever the flags say: the layout does not move with them); the screened tiled
    // product (fp32, on request) keeps its header and its list of uncertified samples there
    const size_t wscreen_bytes = L.variant == KMX_VARIANT_MFMA_WIDE ? kmx_wide_screen_bytes(n, d, k)
                                 : L.gemm_screen                    ? kmx_gemm_screen_bytes(n)
                                                                    : 0;
    L.off_partial = L.off_wscreen + kmx_align256(wscreen_bytes);
    // the matrix-core path accumulates into gsum and needs no per-workgroup partials
    const bool fixed_point = L.variant == KMX_VARIANT_MFMA || L.variant == KMX_VARIANT_MFMA_WIDE || L.screen64;
    L.partial_bytes = fixed_point ? 0 : (size_t)L.n_partials * items * s;
    // (the few-cluster step: per workgroup the accumulators as they lie in its registers)
    if (L.variant == KMX_VARIANT_FEWK) L.partial_bytes = kmx_fewk_partial_bytes(d, k);
    L.total = L.off_partial + kmx_align256(L.partial_bytes);
    return L;
}

// fp32 matrix-core implementations (lloyd_mfma.hip)
// Fixed-point exponents from max|X_t row|, max|w| and n; clears the fixed-point sums.
int32_t kmx_lloyd_mfma_prepare(const LloydLayout& L, const void* X_t, const void* w, char* ws,
                               int64_t n, int d, int dtype, hipStream_t stream);
int32_t kmx_lloyd_iter_mfma_f32(const LloydLayout& L, const void* X_t, const void* w,
                                const void* centroids_t, void* new_centroids_t,
                                const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                                uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                                hipStream_t stream, hipEvent_t* events);
int32_t kmx_assign_labels_mfma_f32(const LloydLayout& L, const void* X_t, const void* centroids_t,
                                   uint32_t* labels, char* ws, int64_t n, int d, int k,
                                   hipStream_t stream);
// Whether the screened fused step finishes the iteration itself (its last workgroup) instead of
// a finalisation launch; 0 restores the separate launch for comparison.
#ifndef KMX_SCR_FUSE_TAIL
#define KMX_SCR_FUSE_TAIL 1
#endif
// screened fused step (lloyd_mfma_screen.hip); `uncertain_count`: one word for the number of
// samples evaluated in fp32
int32_t kmx_lloyd_step_mfma_screen(const void* X_t, const void* w, const void* centroids_t,
                                   const uint32_t* labels_prev, uint32_t* labels,
                                   kmx_lloyd_status* status, const unsigned int* absmax,
                                   const int* q_exp, unsigned long long* gsum,
                                   uint32_t* uncertain_count, const float* norms, int64_t n, int d,
                                   int k, int wgs_per_cu, hipStream_t stream, const LloydTail<float>* tail);
// the same on fp64 inputs: labels screened on the fp16 matrix cores from the inputs rounded to
// fp32, uncertified samples and sums in fp64
int32_t kmx_lloyd_step_mfma_screen_f64(const void* X_t, const void* w, const void* centroids_t,
                                       const uint32_t* labels_prev, uint32_t* labels,
                                       kmx_lloyd_status* status, const unsigned int* absmax,
                                       const int* q_exp, unsigned long long* gsum,
                                       uint32_t* uncertain_count, const float* norms, int64_t n, int d,
                                       int k, int wgs_per_cu, hipStream_t stream, const LloydTail<double>* tail);
int32_t kmx_lloyd_iter_mfma_screen_f64(const LloydLayout& L, const void* X_t, const void* w,
                                       const void* centroids_t, void* new_centroids_t,
                                       const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                                       uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                                       hipStream_t stream, hipEvent_t* events);
int32_t kmx_assign_labels_mfma_screen_f64(const void* X_t, const void* centroids_t, uint32_t* labels, int64_t n,
                                          int d, int k, int wgs_per_cu, hipStream_t stream);
int32_t kmx_assign_labels_fewk(const void* X_t, const void* centroids_t, const void* half_norms, uint32_t* labels,
                               int64_t n, int d, int k, hipStream_t stream);
int32_t kmx_lloyd_iter_fewk(const LloydLayout& L, const void* X_t, const void* X_rowmajor, const void* w,
                            const void* centroids_t, void* new_centroids_t, const uint32_t* labels_prev,
                            uint32_t* labels, void* sizes, uint32_t* empty_clusters, char* ws, int64_t n, int d,
                            int k, hipStream_t stream, hipEvent_t* events);
// labels only, screened the same way (scale from the centroids, norms taken per tile)
int32_t kmx_assign_labels_mfma_screen(const void* X_t, const void* centroids_t, uint32_t* labels,
                                      int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream);
int32_t kmx_assign_labels_inertia_mfma_screen(const void* X_t, const void* w, const void* centroids_t,
                                              uint32_t* labels, double* inertia_partial, int* n_partials,
                                              int64_t n, int d, int k, int wgs_per_cu, hipStream_t stream);
// out[0] = sum of `count` fp64 partial sums, in order (inertia_distances.hip)
int32_t kmx_inertia_total_launch(const double* partial, int count, void* out, int32_t dtype, hipStream_t stream);
int32_t kmx_sample_norms(const void* X_t, float* norms, int64_t n, int d, int dtype, hipStream_t stream);
int32_t kmx_screen_scores_impl(const float* X_t, const float* centroids_t, float* scores,
                               float* bounds, float* half_norms, float* scale, unsigned int* scratch,
                               int64_t n, int d, int k, hipStream_t stream);
int32_t kmx_wide_screen_scale_from_centroids(const void* centroids_t, unsigned int* absmax, int d, int k,
                                             hipStream_t stream);
// labels only through the wide screen: bytes of extra workspace (0: not available), and the pass
size_t kmx_assign_wide_screen_bytes(int64_t n, int d, int k, uint32_t flags);
int32_t kmx_assign_labels_wide_screen_f32(const LloydLayout& L, const void* X_t, const void* centroids_t,
                                          uint32_t* labels, char* ws, char* extra, int64_t n, int d,
                                          int k, hipStream_t stream);
// (labels_prev, status, counts, ranks all null: labels only)
int32_t kmx_lloyd_wide_screen_count(const void* X_t, const void* centroids_t,
                                    const unsigned int* absmax, char* area,
                                    const uint32_t* labels_prev, uint32_t* labels,
                                    kmx_lloyd_status* status, int* counts, int* ranks, int64_t n,
                                    int d, int k, hipStream_t stream);
// wide-sample variant (lloyd_mfma_wide.hip): the fused step only; the reduction and
// finalisation kernels of lloyd.hip follow it
int32_t kmx_lloyd_step_mfma_wide_f32(const LloydLayout& L, const void* X_t, const void* X_rowmajor,
                                     const void* w, const void* centroids_t,
                                     const uint32_t* labels_prev, uint32_t* labels, char* ws,
                                     int64_t n, int d, int k, hipStream_t stream);
int32_t kmx_assign_labels_mfma_wide_f32(const LloydLayout& L, const void* X_t,
                                        const void* centroids_t, uint32_t* labels, char* ws,
                                        int64_t n, int d, int k, hipStream_t stream);

// fp64 matrix-core fused step (lloyd_mfma_f64.hip): fills partial[0 .. grid) like the
// vector-ALU kernels with LDS accumulators; `update` false = labels only
int kmx_mfma_f64_grid(int64_t n, int d, int wgs_per_cu, int cols, int max_slots);
int32_t kmx_lloyd_step_mfma_f64(const void* X_t, const void* w, const void* centroids_t,
                                const void* half_norms, const uint32_t* labels_prev,
                                uint32_t* labels, void* partial, kmx_lloyd_status* status,
                                int64_t n, int d, int k, bool update, int wgs_per_cu, int cols,
                                int max_slots, hipStream_t stream);
