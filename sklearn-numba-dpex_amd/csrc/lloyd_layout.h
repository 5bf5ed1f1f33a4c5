// Workspace layout and kernel selection of the Lloyd iteration, shared by the vector-ALU
// and MFMA implementations.
#pragma once

#include "kmx_common.h"

constexpr int KMX_VARIANT_STREAM = 0;    // wide samples: features re-read per centroid window
constexpr int KMX_VARIANT_REGISTER = 1;  // samples held in registers, centroids in SGPRs
constexpr int KMX_VARIANT_MFMA = 3;      // fp32 distances on the matrix cores

constexpr int KMX_ACC_LDS = 1;
constexpr int KMX_ACC_GLOBAL = 2;

constexpr int KMX_MAX_PARTIALS = 1024;          // upper bound on fused-step workgroups
constexpr size_t KMX_LDS_ACC_LIMIT = 40000;     // bytes of LDS accumulators per workgroup
constexpr size_t KMX_GLOBAL_COPIES_BYTES = 64u << 20;

struct LloydLayout {
    int dpad;            // features per packed centroid row (multiple of 4, zero padded)
    int variant;         // KMX_VARIANT_*
    int acc_mode;        // KMX_ACC_*
    int n_partials;      // slots in `partial` (workgroups for LDS mode, copies for global mode)
    size_t off_status, off_cpack, off_half, off_shift, off_partial;
    size_t partial_bytes;
    size_t total;
    // Workgroups of the fused step: four per compute unit, never more than the partial slots.
    int grid_cap(int cus) const {
        const int g = 4 * cus;
        return g < n_partials ? g : n_partials;
    }
};

static inline int lloyd_reg_samples_per_thread(int d, int dtype) {
    if (dtype == KMX_F32) return d <= 16 ? 4 : (d <= 32 ? 2 : 1);
    return d <= 16 ? 2 : 1;
}

// Environment override for experiments: KMX_LLOYD_VARIANT = stream | register | mfma.
int kmx_forced_variant();

static inline LloydLayout lloyd_layout(int64_t n, int d, int k, int dtype) {
    (void)n;
    LloydLayout L;
    const size_t s = kmx_dtype_size(dtype);
    L.dpad = (d + 3) & ~3;
    const size_t items = (size_t)(d + 1) * k;
    const bool reg_ok = (dtype == KMX_F32) ? d <= 64 : d <= 32;
    L.variant = reg_ok ? KMX_VARIANT_REGISTER : KMX_VARIANT_STREAM;
    const int forced = kmx_forced_variant();
    if (forced == KMX_VARIANT_STREAM) L.variant = KMX_VARIANT_STREAM;
    if (forced == KMX_VARIANT_REGISTER && reg_ok) L.variant = KMX_VARIANT_REGISTER;
    if (items * s <= KMX_LDS_ACC_LIMIT) {
        L.acc_mode = KMX_ACC_LDS;
        L.n_partials = KMX_MAX_PARTIALS;
    } else {
        L.acc_mode = KMX_ACC_GLOBAL;
        size_t copies = KMX_GLOBAL_COPIES_BYTES / (items * s);
        if (copies < 1) copies = 1;
        if (copies > 32) copies = 32;
        L.n_partials = (int)copies;
    }
    L.off_status = 0;
    L.off_cpack = kmx_align256(sizeof(kmx_lloyd_status));
    L.off_half = L.off_cpack + kmx_align256((size_t)k * L.dpad * s);
    L.off_shift = L.off_half + kmx_align256((size_t)k * s);
    L.off_partial = L.off_shift + kmx_align256((size_t)kmx_cdiv(k, 256) * sizeof(double));
    L.partial_bytes = (size_t)L.n_partials * items * s;
    L.total = L.off_partial + kmx_align256(L.partial_bytes);
    return L;
}

// fp32 matrix-core implementations (lloyd_mfma.hip)
int32_t kmx_lloyd_iter_mfma_f32(const LloydLayout& L, const void* X_t, const void* w,
                                const void* centroids_t, void* new_centroids_t,
                                const uint32_t* labels_prev, uint32_t* labels, void* sizes,
                                uint32_t* empty_clusters, char* ws, int64_t n, int d, int k,
                                hipStream_t stream, hipEvent_t* events);
int32_t kmx_assign_labels_mfma_f32(const LloydLayout& L, const void* X_t, const void* centroids_t,
                                   uint32_t* labels, char* ws, int64_t n, int d, int k,
                                   hipStream_t stream);
