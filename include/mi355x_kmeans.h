/*
 * mi355x_kmeans.h - C ABI of libmi355x_kmeans.so (HIP kernels for gfx950).
 *
 * One entry point per kernel family of the reference KMeans engine
 * (soda-inria/sklearn-numba-dpex).  The reference has no FFI of its own: its kernels are
 * numba_dpex JIT functions created by `make_*` factories and launched from
 * sklearn_numba_dpex/kmeans/drivers.py.  Each declaration below cites the factory or driver
 * code it replaces (paths relative to the reference's sklearn_numba_dpex/ directory).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless its name ends in `_host`.
 *   - Data layout is the reference's: X_t is (n_features, n_samples) row-major, centroids_t
 *     is (n_features, n_clusters) row-major (kmeans/drivers.py:43-53, kmeans/engine.py:88-98).
 *   - `dtype`: KMX_F32 or KMX_F64, the type of every `void*` floating array of the call.
 *   - Labels are uint32, kmeans++ indices int32, top-k indices int64 (as in the reference).
 *   - Outputs and workspaces are allocated by the caller; `*_workspace_bytes` give sizes.
 *     No entry point allocates or frees device memory.
 *   - `stream` is a hipStream_t (NULL = default stream).  Calls only enqueue work; none
 *     synchronises except kmx_lloyd_status_read.
 *   - Return value: 0 on success, a negative KMX_ERR_* for rejected arguments, or a positive
 *     hipError_t reported by the runtime.  Nothing throws or exits.
 *   - Calls that share a workspace must be issued on one stream (or otherwise ordered).
 *   - The library keeps no selection state and reads no environment variable: which kernel
 *     runs follows from the shape and from the caller's `flags` (KMX_FLAG_*) alone.
 */
#ifndef MI355X_KMEANS_H
#define MI355X_KMEANS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KMX_F32 0
#define KMX_F64 1

#define KMX_OK 0
#define KMX_ERR_NULL_POINTER (-1)
#define KMX_ERR_BAD_SHAPE (-2)      /* n, d, k, rows, cols <= 0 or inconsistent            */
#define KMX_ERR_BAD_DTYPE (-3)
#define KMX_ERR_WORKSPACE (-4)      /* workspace smaller than *_workspace_bytes()          */
#define KMX_ERR_BAD_ARGUMENT (-5)   /* k > n for top-k, unknown op code, ...               */
#define KMX_ERR_UNSUPPORTED (-6)    /* shape outside what a specialised kernel covers      */

#define KMX_ERR_BAD_PLAN (-7)       /* kmx_lloyd_plan not made by kmx_lloyd_plan_init, or edited */

#define KMX_ABI_VERSION 3
int32_t kmx_abi_version(void);
const char* kmx_error_string(int32_t code);

/* ------------------------------------------------------------------------------------ *
 * Lloyd iteration                                                                       *
 * ------------------------------------------------------------------------------------ */

/* Loop state kept on the device (first bytes of the Lloyd workspace). */
#define KMX_RUNNING 0
#define KMX_CONVERGED_STRICT 1   /* no label changed between two successive iterations  */
#define KMX_CONVERGED_TOL 2      /* shift_sum <= tol                                    */
#define KMX_MAX_ITER 3
#define KMX_NEED_RELOCATION 4    /* empty clusters found: host must relocate + finalize */

typedef struct kmx_lloyd_status {
    int32_t n_iter;       /* iterations completed                                          */
    int32_t state;        /* KMX_RUNNING ...                                               */
    int32_t n_empty;      /* empty clusters found by the last reduction                    */
    uint32_t n_changed;   /* labels that differ from the previous iteration's              */
    double shift_sum;     /* sum_c ||old_c - new_c||^2 of the last finalised iteration     */
    double tol;           /* loop runs while shift_sum > tol                               */
    int32_t max_iter;
    uint32_t ticket;      /* internal: block counter of the reduction kernel               */
    double max_sq_dist;   /* scratch for the relocation guard                              */
    int64_t reserved[2];
} kmx_lloyd_status;       /* 64 bytes */

/* Kernel selection: `flags` of kmx_lloyd_plan_init and kmx_assign_labels.  0 leaves every
 * choice to the library (the fastest kernel it has for the shape).  The reference has no
 * counterpart: its kernels are specialised by the JIT from the shape alone
 * (kmeans/drivers.py:103-135). */
#define KMX_FLAG_PATH_MASK 0x0000000fu
#define KMX_FLAG_PATH_AUTO 0x0u
#define KMX_FLAG_PATH_STREAM 0x1u      /* features re-read per centroid window                */
#define KMX_FLAG_PATH_REGISTER 0x2u    /* samples in registers, vector ALU                    */
#define KMX_FLAG_PATH_MFMA 0x3u        /* matrix cores wherever the shape allows              */
#define KMX_FLAG_PATH_GEMM 0x4u        /* tiled matrix-core labels + bucketed sums (any shape) */
#define KMX_FLAG_LABELS_MASK 0x00000030u
#define KMX_FLAG_LABELS_AUTO 0x00u
#define KMX_FLAG_LABELS_F32 0x10u      /* no fp16 screen: every product in the input type     */
#define KMX_FLAG_LABELS_SCREEN 0x20u   /* fp16 screen + fp32 certificate wherever it fits (also the tiled product) */
#define KMX_FLAG_WGS_PER_CU(x) (((uint32_t)(x) & 0xfu) << 8)  /* 1..8 workgroups per CU; 0: default */
#define KMX_FLAG_COLS(x) (((uint32_t)(x) & 0x7u) << 12)       /* 2 | 4 sample columns per lane; 0: default */

/* What kmx_lloyd_init / kmx_lloyd_iter / kmx_lloyd_finalize run for one problem: the shape, the
 * caller's flags, the kernel variant chosen from them and the workspace the variant needs.
 * Plain host memory owned by the caller, filled by kmx_lloyd_plan_init and passed unchanged to
 * the other calls: the workspace layout is a function of the plan, so the calls of one fit
 * cannot disagree about it.  A plan that was not made by kmx_lloyd_plan_init of this library
 * version, or whose fields were edited afterwards, is rejected with KMX_ERR_BAD_PLAN. */
typedef struct kmx_lloyd_plan {
    uint32_t magic;
    int32_t abi_version;
    int64_t n;
    int32_t d;
    int32_t k;
    int32_t dtype;
    uint32_t flags;
    int32_t variant;           /* 10 * path + accumulation, see kmx_lloyd_kernel_variant      */
    int32_t reserved;
    uint64_t workspace_bytes;  /* bytes of device memory kmx_lloyd_init and the others need   */
    uint64_t check;            /* over the fields above                                       */
} kmx_lloyd_plan;              /* 56 bytes */

/* Fills `plan` for n samples, d features, k clusters.  KMX_ERR_BAD_SHAPE, KMX_ERR_BAD_DTYPE or
 * KMX_ERR_BAD_ARGUMENT (flags that name no choice).  Host only: no device work.
 * Replaces the kernel factories' specialisation on the shape, kmeans/drivers.py:103-135. */
int32_t kmx_lloyd_plan_init(kmx_lloyd_plan* plan, int64_t n, int32_t d, int32_t k, int32_t dtype,
                            uint32_t flags);

/* plan.workspace_bytes / plan.variant without a plan (0 / a negative code for bad arguments). */
size_t kmx_lloyd_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags);

/* Resets the loop state, packs the initial centroids (+ their half squared norms), clears
 * the accumulators and, for the fixed-point accumulation of the fp32 matrix-core path, takes
 * max|x| per feature and max|w| (one pass over X_t and sample_weight).
 * Replaces the set-up part of lloyd(), kmeans/drivers.py:146-184. */
int32_t kmx_lloyd_init(const kmx_lloyd_plan* plan, void* workspace, size_t workspace_bytes,
                       const void* X_t, const void* sample_weight, const void* centroids_t,
                       int32_t max_iter, double tol, void* stream);

/* One Lloyd iteration, enqueued as two kernels (three for shapes whose partial sums do not
 * fit in LDS):
 *   (1) fused step: pseudo distances 0.5||c||^2 - <x,c>, argmin (lowest index wins ties),
 *       label write, changed-label count, per-workgroup partial sums of w*x and w;
 *   (2) reduction of the partial sums, empty-cluster list (ascending), and - when no cluster
 *       is empty - division by the cluster sizes, centroid shift and convergence test.
 * Does nothing if the state is not KMX_RUNNING, so iterations may be enqueued ahead of the
 * host's next look at the status.
 * Replaces make_lloyd_single_step_fixed_window_kernel (kmeans/kernels/lloyd_single_step.py:35-424),
 * make_reduce_centroid_data_kernel (kmeans/kernels/utils.py:113-195),
 * make_half_l2_norm_2d_axis0_kernel, make_initialize_to_zeros_kernel,
 * make_broadcast_division_1d_2d_axis0_kernel (common/kernels.py:38-145),
 * make_centroid_shifts_kernel (kmeans/kernels/utils.py:79-110) and the loop body of
 * lloyd(), kmeans/drivers.py:188-343.
 *   X_rowmajor       IN   (n, d)  optional (may be NULL) row-major copy of the same data; used
 *                                 by the wide fp32 path (plan.variant == 42), which then sums
 *                                 each cluster's rows instead of issuing one global atomic per
 *                                 (sample, feature), and by the bucketed sums (plan.variant
 *                                 63, 53, 13 or 3), which read whole rows from it instead
 *                                 of gathering the feature-major array
 *   centroids_t      IN   (d, k)  centroids the labels are computed from: the array given to
 *                                 kmx_lloyd_init for the first iteration, then the
 *                                 new_centroids_t of the previous one (the workspace holds a
 *                                 packed copy and the half squared norms of exactly those)
 *   new_centroids_t  OUT  (d, k)  un-normalised sums if relocation is needed, else new centroids
 *   labels_prev      IN   (n)     labels of the previous iteration: from the second iteration on
 *                                 exactly the array the previous kmx_lloyd_iter of this workspace
 *                                 wrote as `labels` (the callers ping-pong two arrays).  Besides
 *                                 the count of changed labels, variants 61 and 71 build on it: once few
 *                                 labels change it no longer rebuilds its integer sums but moves
 *                                 every sample that changes cluster from the old sum to the new one
 *   labels           OUT  (n)
 *   cluster_sizes    OUT  (k)     sum of weights per cluster
 *   empty_clusters   OUT  (k)     ids of empty clusters, ascending, first status.n_empty valid */
int32_t kmx_lloyd_iter(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                       const void* sample_weight, const void* centroids_t, void* new_centroids_t,
                       const uint32_t* labels_prev, uint32_t* labels, void* cluster_sizes,
                       uint32_t* empty_clusters, void* workspace, size_t workspace_bytes,
                       void* stream);

/* kmx_lloyd_iter with HIP events recorded on `stream` around each of its kernels.  Waits for
 * the iteration and writes the three durations in milliseconds (fused step, reduction,
 * finalisation) to kernel_ms_host[0..2].  For benchmarks and profiling; it has no
 * counterpart in the reference, whose benchmark only times a whole fit
 * (benchmark/kmeans.py:163-165). */
int32_t kmx_lloyd_iter_timed(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                             const void* sample_weight, const void* centroids_t,
                             void* new_centroids_t, const uint32_t* labels_prev, uint32_t* labels,
                             void* cluster_sizes, uint32_t* empty_clusters, void* workspace,
                             size_t workspace_bytes, void* stream, float* kernel_ms_host);

/* kmx_lloyd_iter with the same events, without waiting: the launch is enqueued like any other and
 * its four events are kept by the library (up to 1 024 launches: KMX_ERR_UNSUPPORTED beyond), so
 * that a benchmark can time every launch of a stream of back-to-back iterations instead of
 * iterations that each wait for the host.  kmx_lloyd_trace_collect waits for the launches
 * enqueued so far, writes the mean (and, if kernel_ms_min is not NULL, the minimum) duration in
 * milliseconds of each of the three kernel groups over them, their number, and forgets them.
 * Not for concurrent fits: the list is one per process.  No counterpart in the reference
 * (benchmark/kmeans.py:163-165 times whole fits). */
int32_t kmx_lloyd_iter_traced(const kmx_lloyd_plan* plan, const void* X_t, const void* X_rowmajor,
                              const void* sample_weight, const void* centroids_t,
                              void* new_centroids_t, const uint32_t* labels_prev, uint32_t* labels,
                              void* cluster_sizes, uint32_t* empty_clusters, void* workspace,
                              size_t workspace_bytes, void* stream);
int32_t kmx_lloyd_trace_collect(float* kernel_ms_mean, float* kernel_ms_min, int32_t* n_launches);

/* Second half of (2) alone, for the iteration that stopped with KMX_NEED_RELOCATION after
 * the host has relocated the empty clusters: sums / sizes, shift, convergence test, state
 * back to KMX_RUNNING (or a terminal state).  kmeans/drivers.py:275,326-343. */
int32_t kmx_lloyd_finalize(const kmx_lloyd_plan* plan, const void* centroids_t,
                           void* new_centroids_t, const void* cluster_sizes, void* workspace,
                           size_t workspace_bytes, void* stream);

/* Copies the status to host memory and waits for it (the only synchronising call). */
int32_t kmx_lloyd_status_read(const void* workspace, kmx_lloyd_status* status_host, void* stream);

/* Kernel variants 61 and 71 only (labels screened on the fp16 matrix cores): number of samples
 * whose label the screen of the last completed iteration could not certify and that were
 * evaluated in the input type instead; 0 for the other variants.  Synchronises the stream.
 * It has no counterpart in the reference (diagnostics). */
int32_t kmx_lloyd_recheck_count(const kmx_lloyd_plan* plan, const void* workspace,
                                uint32_t* count_host, void* stream);

/* Diagnostics of kernel variant 61, for tests of its certificate: the approximate scores
 * <x, c> - 0.5||c||^2 exactly as the fused step forms them on the fp16 matrix cores (same
 * power-of-two scaling, same two-part fp16 split, same MFMA sequence), in scaled units
 * (x * scale, c * scale): scores (k, n), the per-sample error bound bounds (n) the step
 * compares half the best-to-second gap with, the fp32 0.5||c * scale||^2 it starts from
 * half_norms (k), and scale (1).  fp32 only; d <= 256 and k small enough for the operands of
 * all centroids to fit 64 KB of LDS (the wide path, variant 42, uses the same arithmetic),
 * else KMX_ERR_UNSUPPORTED; scratch: 256 bytes of device memory.
 * It has no counterpart in the reference (diagnostics). */
int32_t kmx_screen_scores(const void* X_t, const void* centroids_t, float* scores, float* bounds,
                          float* half_norms, float* scale, void* scratch, int64_t n, int32_t d,
                          int32_t k, void* stream);

/* Which fused-step kernel kmx_lloyd_iter uses for a shape and flags, as 10 * path + accumulation:
 * path 0 = streaming vector-ALU step (wide samples, up to 16 clusters), 1 = register-resident
 * samples (vector ALU), 3 = MFMA (fp32) with the centroids resident in LDS, 4 = MFMA (fp32)
 * with samples in registers and centroids streamed (more than 256 clusters), 5 = MFMA (fp64)
 * with the centroids resident in LDS, 6 = labels by a tiled matrix-core product (any shape,
 * fp32 and fp64), 8 = fp32 with up to 16 clusters and 65 .. 1792 features: a tile of samples on chip
 * serves labels and sums on the matrix cores, X read once; accumulation 1 = workgroup-private LDS accumulators, 2 = global sums,
 * 3 = labels only, then sums by a kernel of their own (per bucket of samples sorted by label,
 * or, fp32, straight from the labels into fixed-point accumulators in LDS where those of every
 * cluster fit).  61 is path 3 with the labels screened on the fp16 matrix cores; 71 is the same
 * step on fp64 inputs (rows rounded to fp32 for the screen, the samples it cannot certify on the
 * fp64 matrix cores, sums from the fp64 rows), chosen over 51 wherever its operands fit the LDS. */
int32_t kmx_lloyd_kernel_variant(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags);

/* 1 when the plan's kernels read the row-major copy of X that kmx_lloyd_iter takes as
 * `X_rowmajor` (the wide fp32 step always; the sums per bucket of samples and the few-cluster step
 * optionally, NULL makes them read the feature-major array), 0 when they ignore it, negative: error.  Host only.
 * Has no counterpart in the reference, whose kernels read one layout (the transposed copy made
 * in sklearn_numba_dpex/kmeans/engine.py:88-98): it lets a caller skip the second copy of X. */
int32_t kmx_lloyd_plan_reads_rowmajor(const kmx_lloyd_plan* plan);

/* ------------------------------------------------------------------------------------ *
 * Labels, inertia, distances                                                            *
 * ------------------------------------------------------------------------------------ */

size_t kmx_assign_workspace_bytes(int32_t d, int32_t k, int32_t dtype);

/* The workspace with which kmx_assign_labels takes its fastest path for n samples: wide fp32
 * shapes screen the labels on the fp16 matrix cores and need room for a list of samples.  Never
 * smaller than kmx_assign_workspace_bytes, which always suffices.  It has no counterpart in the
 * reference (workspaces belong to this library). */
size_t kmx_assign_workspace_bytes_for(int64_t n, int32_t d, int32_t k, int32_t dtype, uint32_t flags);

/* labels[i] = argmin_c (0.5||c||^2 - <x_i, c>).  Replaces
 * make_label_assignment_fixed_window_kernel (kmeans/kernels/compute_labels.py:18-185) and the
 * half-norm call before it (kmeans/drivers.py:657-669). */
int32_t kmx_assign_labels(const void* X_t, const void* centroids_t, uint32_t* labels,
                          void* workspace, size_t workspace_bytes, int64_t n, int32_t d,
                          int32_t k, int32_t dtype, uint32_t flags, void* stream);

/* out[i] = w_i * sum_f (x_fi - c_f,label_i)^2, features in order; sample_weight may be NULL
 * for unit weights (the relocation pass).  Replaces make_compute_inertia_kernel
 * (kmeans/kernels/compute_inertia.py:8-42). */
int32_t kmx_per_sample_inertia(const void* X_t, const void* sample_weight, const void* centroids_t,
                               const uint32_t* labels, void* out, int64_t n, int32_t d,
                               int32_t k, int32_t dtype, void* stream);

/* out_total[0] = sum_i w_i * ||x_i - c_label_i||^2: the per-sample kernel with the sum folded in
 * (fp64 totals per workgroup in `workspace`, added in order by a second small launch), so the
 * n per-sample values are neither written nor read back.  Replaces compute_inertia_kernel
 * followed by the sum reduction at the end of a fit and in get_labels_inertia
 * (kmeans/drivers.py:379-391, 674-697; kmeans/kernels/compute_inertia.py:9-42). */
size_t kmx_inertia_workspace_bytes(int64_t n);
int32_t kmx_inertia(const void* X_t, const void* sample_weight, const void* centroids_t,
                    const uint32_t* labels, void* out_total, void* workspace,
                    size_t workspace_bytes, int64_t n, int32_t d, int32_t k, int32_t dtype,
                    void* stream);

/* Labels and the weighted inertia of that labelling in one call: kmx_assign_labels followed by
 * kmx_inertia, except that where the screened label kernel applies (fp32, d <= 64) X is read
 * once - the kernel sums w_i ||x_i - c_label_i||^2 of its samples on the way.  sample_weight may
 * be NULL (unit weights).  out_total: one element of the compute dtype.  Replaces
 * get_labels_inertia with with_inertia=True and the final E-step of a fit
 * (kmeans/drivers.py:356-391, 630-699). */
size_t kmx_assign_inertia_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t dtype,
                                          uint32_t flags);
int32_t kmx_assign_labels_inertia(const void* X_t, const void* sample_weight,
                                  const void* centroids_t, uint32_t* labels, void* out_total,
                                  void* workspace, size_t workspace_bytes, int64_t n, int32_t d,
                                  int32_t k, int32_t dtype, uint32_t flags, void* stream);

/* distances_t (k, n): sqrt(sum_f (c_f - x_f)^2).  Replaces
 * make_compute_euclidean_distances_fixed_window_kernel
 * (kmeans/kernels/compute_euclidean_distances.py:15-161). */
int32_t kmx_euclidean_distances(const void* X_t, const void* centroids_t, void* distances_t,
                                int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream);

/* Moves each listed empty cluster onto a far sample, on the un-normalised sums:
 * sums[:, old] -= w*x, sums[:, empty] = w*x, sizes likewise; per_sample_inertia (may be NULL)
 * of the moved sample is zeroed.  Replaces make_relocate_empty_clusters_kernel
 * (kmeans/kernels/utils.py:11-76). */
int32_t kmx_relocate_empty_clusters(const void* X_t, const void* sample_weight,
                                    const uint32_t* labels, const int64_t* far_samples,
                                    const uint32_t* empty_clusters, int32_t n_relocated,
                                    void* per_sample_inertia, void* sums_t, void* cluster_sizes,
                                    int64_t n, int32_t d, int32_t k, int32_t dtype, void* stream);

/* ------------------------------------------------------------------------------------ *
 * kmeans++ seeding                                                                      *
 * ------------------------------------------------------------------------------------ */

/* Host-side generator of the sampler's draws (no device work, callable without a GPU).
 * kmx_rng_init_states fills `states` (n_states, 2) with xoroshiro128++ states: SplitMix64
 * seeding of the first one, then `subsequence_start` jumps of 2^64 steps, every further state
 * one more jump ahead.  kmx_rng_next_raw advances every state n_steps times and writes the raw
 * 64-bit outputs to `out` (n_steps, n_states), step-major.  Replace create_xoroshiro128pp_states
 * and the make_rand_uniform_kernel_func stream (common/random.py:124-292); the uint64 -> [0, 1)
 * conversion (:78-104) stays with the caller. */
int32_t kmx_rng_init_states(uint64_t seed, int32_t n_states, int32_t subsequence_start,
                            uint64_t* states);
int32_t kmx_rng_next_raw(uint64_t* states, int32_t n_states, int32_t n_steps, uint64_t* out);

size_t kmx_kpp_workspace_bytes(int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype);

/* closest[i] = w_i ||x_i - x_start||^2, centers_t[:, 0] = x_start, center_indices[0] = start,
 * and the per-block partial potentials.  Replaces make_kmeansplusplus_init_kernel
 * (kmeans/kernels/kmeans_plusplus.py:16-58) + the potential reduction (kmeans/drivers.py:844). */
int32_t kmx_kpp_init(const void* X_t, const void* sample_weight, int32_t start_index,
                     void* centers_t, int32_t* center_indices, void* workspace,
                     size_t workspace_bytes, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                     int32_t dtype, uint32_t flags, void* stream);

/* Which sampler kmx_kpp_sample_candidates and kmx_kpp_run use (`flags`).
 * KMX_KPP_SAMPLER_SCAN (default): candidate t = first j with (inclusive fp64 scan of closest)_j
 * >= uniforms[t] * total, clipped to [0, n-1]: a two-level search over the block potentials
 * already held in the workspace.
 * KMX_KPP_SAMPLER_LITERAL: the reference's sampler statement by statement
 * (kmeans/kernels/kmeans_plusplus.py:79-100): running sum of closest in the compute dtype from
 * sample 0, first j whose running sum reaches T(uniforms[t]) * T(total), clipped to n-1; a
 * trial with uniforms[t] * total <= 0 gets n-1 (the reference leaves -1 there, which its next
 * kernel reads as an index from the end).  With the same flag kmx_kpp_init and kmx_kpp_step
 * round the product and the sum of every squared difference separately, as the reference's two
 * statements do (the default is one fused multiply-add: the running sum in the compute dtype
 * turns a last-bit difference in one distance into another candidate), and kmx_kpp_step
 * compares the trial potentials after rounding them to the compute dtype.  One wave walks the
 * array: about 8 ns per sample and centre, for parity checks against the reference, not for
 * speed. */
#define KMX_KPP_SAMPLER_SCAN 0x0u
#define KMX_KPP_SAMPLER_LITERAL 0x1u

/* Replaces make_sample_center_candidates_kernel (kmeans/kernels/kmeans_plusplus.py:61-103).
 *   uniforms_for_step  IN  (n_trials) doubles in [0, 1)
 *   candidates         OUT (n_trials) int32, may be NULL (they stay in the workspace)
 *   flags              KMX_KPP_SAMPLER_*; anything else: KMX_ERR_BAD_ARGUMENT */
int32_t kmx_kpp_sample_candidates(const void* X_t, const double* uniforms_for_step,
                                  int32_t* candidates, void* workspace, size_t workspace_bytes,
                                  int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype,
                                  uint32_t flags, void* stream);

/* For every candidate t and sample i: min(w_i ||x_i - x_cand_t||^2, closest_i), row sums,
 * argmin over t (lowest t wins ties), closest <- best row, centers_t[:, c] <- x_best,
 * center_indices[c] <- best candidate.  Replaces
 * make_kmeansplusplus_single_step_fixed_window_kernel (kmeans/kernels/kmeans_plusplus.py:106-262),
 * the axis-1 sum and argmin reductions (common/reductions.py) and kmeans/drivers.py:886-908. */
int32_t kmx_kpp_step(const void* X_t, const void* sample_weight, int32_t center_slot,
                     void* centers_t, int32_t* center_indices, void* workspace,
                     size_t workspace_bytes, int64_t n, int32_t d, int32_t k, int32_t n_trials,
                     int32_t dtype, uint32_t flags, void* stream);

/* The whole seeding (init, then k-1 x [sample, step]) with no host round trip.
 *   uniforms  IN (k-1, n_trials) doubles: row c-1 holds what trial t draws for centre c.
 *   flags     KMX_KPP_SAMPLER_*
 * Replaces kmeans_plusplus(), kmeans/drivers.py:735-910. */
int32_t kmx_kpp_run(const void* X_t, const void* sample_weight, const double* uniforms,
                    int32_t start_index, void* centers_t, int32_t* center_indices,
                    void* workspace, size_t workspace_bytes, int64_t n, int32_t d, int32_t k,
                    int32_t n_trials, int32_t dtype, uint32_t flags, void* stream);

/* Views into the kmeans++ workspace, for tests: closest (n) in `dtype`, potentials
 * (n_trials) doubles of the last step, candidates (n_trials) int32. */
void* kmx_kpp_closest_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype);
double* kmx_kpp_potentials_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype);
int32_t* kmx_kpp_candidates_ptr(void* workspace, int64_t n, int32_t d, int32_t k, int32_t n_trials, int32_t dtype);

/* ------------------------------------------------------------------------------------ *
 * Shared kernels (the reference's common/ directory)                                    *
 * ------------------------------------------------------------------------------------ */

size_t kmx_sum_workspace_bytes(int64_t rows, int64_t cols);

/* out[r] = sum_c f(in[r, c]) with f = identity or square (first pass only).  Replaces
 * make_sum_reduction_2d_kernel with axis=1 and the 1-D form (common/reductions.py:214-460,
 * 643-890).  Accumulates in fp64, fixed order: results are reproducible run to run. */
int32_t kmx_sum_rows(const void* in, void* out, int64_t rows, int64_t cols, int32_t square,
                     void* workspace, size_t workspace_bytes, int32_t dtype, void* stream);

/* kmx_sum_rows for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same result,
 * with the per-workgroup partial sums in a 128 KiB array that is part of the library's device
 * image instead of a caller-provided workspace.  It has no counterpart in the reference.
 * Calls no hipMalloc / hipFree or any allocating routine.  Limit: rows <= 64 (else
 * KMX_ERR_UNSUPPORTED); cols unlimited.  Each GPU has ONE such array, shared by every call
 * on that GPU: calls that overlap in time on one GPU (different streams, different threads)
 * race on it and must be ordered by the caller.  Nothing in it needs to start at zero. */
int32_t kmx_sum_rows_static(const void* in, void* out, int64_t rows, int64_t cols, int32_t square,
                            int32_t dtype, void* stream);

/* out[c] = sum_r in[r, c].  Replaces the axis=0 form (common/reductions.py:462-640). */
int32_t kmx_sum_cols(const void* in, void* out, int64_t rows, int64_t cols, void* workspace,
                     size_t workspace_bytes, int32_t dtype, void* stream);

/* out[0] = index of the smallest value, lowest index on ties.  Replaces
 * make_argmin_reduction_1d_kernel (common/reductions.py:17-209). */
int32_t kmx_argmin(const void* values, int32_t* out, int64_t n, int32_t dtype, void* stream);

/* out[c] = (sum_f a[f, c]^2) / 2.  make_half_l2_norm_2d_axis0_kernel, common/kernels.py:116-145. */
int32_t kmx_half_sq_norms(const void* a_t, void* out, int32_t rows, int32_t cols, int32_t dtype,
                          void* stream);

/* a[r, c] = a[r, c] (op) v[r], op 0 = minus, 1 = plus.
 * make_broadcast_ops_1d_2d_axis1_kernel, common/kernels.py:85-113. */
int32_t kmx_broadcast_rows(void* a, const void* v, int64_t rows, int64_t cols, int32_t op,
                           int32_t dtype, void* stream);

/* a[r, c] /= v[c].  make_broadcast_division_1d_2d_axis0_kernel, common/kernels.py:60-82. */
int32_t kmx_broadcast_div_cols(void* a, const void* v, int64_t rows, int64_t cols, int32_t dtype,
                               void* stream);

/* dst (cols, rows) = the transpose of src (rows, cols), both row-major and distinct.  The
 * reference leaves its transposed copies to the array library (`X.T` through dpctl /
 * `dpt.asarray(..., order="C")`: sklearn_numba_dpex/kmeans/engine.py:88-98,
 * kmeans/drivers.py:43-53); here the ingest of a row-major X and the row-major copy that the
 * bucketed sums read go through this kernel. */
int32_t kmx_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int32_t dtype,
                      void* stream);

/* data[i] = data[i] / divisor.  make_apply_elementwise_func with _divide_by,
 * common/kernels.py:11-36, common/_utils.py:17-33. */
int32_t kmx_divide_by(void* data, int64_t n_items, double divisor, int32_t dtype, void* stream);

/* Zero fill.  make_initialize_to_zeros_kernel, common/kernels.py:38-57. */
int32_t kmx_fill_zero(void* data, int64_t n_bytes, void* stream);

/* out[c] = sum_f (a[f, c] - b[f, c])^2.  make_centroid_shifts_kernel, kmeans/kernels/utils.py:79-110. */
int32_t kmx_centroid_shifts(const void* a_t, const void* b_t, void* out, int32_t d, int32_t k,
                            int32_t dtype, void* stream);

/* Workspace of the top-k entry points for `rows` rows of `n` values: per row a histogram, the
 * k winners and a side buffer for a quarter of the row.  0 for arguments the entry points
 * refuse.  kmx_topk_workspace_bytes is the one-row size that serves either dtype. */
size_t kmx_topk_rows_workspace_bytes(int64_t rows, int64_t n, int32_t k, int32_t dtype);
size_t kmx_topk_workspace_bytes(int64_t n, int32_t k);

/* out_indices (rows, k) = per row of the C-contiguous matrix `values` (rows, n), the indices
 * of its k largest values by radix select (digits of 11 or 10 bits, most significant first, on
 * the order-preserving unsigned image of the floats; -0.0 counts as +0.0, NaNs of positive
 * sign rank above +inf), ordered by descending value then ascending index; of equal values at
 * the threshold the lowest indices are taken.  All rows advance in one chain of launches.  The
 * final ordering compares every pair of winners, k^2 comparisons per row.  Replaces topk_idx
 * (common/topk.py:194-270, 273-527, 540-1123, 1250-1365), whose output order is undefined. */
int32_t kmx_topk_idx_rows(const void* values, int64_t* out_indices, int64_t rows, int64_t n,
                          int32_t k, void* workspace, size_t workspace_bytes, int32_t dtype,
                          void* stream);

/* out_values (rows, k) = the k largest values of each row, descending (the values at the
 * indices kmx_topk_idx_rows returns, bit for bit).  Replaces topk (common/topk.py:112-191,
 * 1127-1247). */
int32_t kmx_topk_values(const void* values, void* out_values, int64_t rows, int64_t n, int32_t k,
                        void* workspace, size_t workspace_bytes, int32_t dtype, void* stream);

/* kmx_topk_idx_rows for one row: topk_idx on a 1-D array (common/topk.py:229-235). */
int32_t kmx_topk_idx(const void* values, int64_t* out_indices, int64_t n, int32_t k,
                     void* workspace, size_t workspace_bytes, int32_t dtype, void* stream);

/* result[0] = 1 if the two labelings are equal up to a permutation of the labels, else 0.
 * mapping: scratch of k int32.  make_is_same_clustering_kernel, kmeans/kernels/utils.py:198-253. */
int32_t kmx_is_same_clustering(const uint32_t* labels1, const uint32_t* labels2, int32_t* mapping,
                               int32_t* result, int64_t n, int32_t k, void* stream);

/* result[0] = number of distinct labels.  seen: scratch of k int32.
 * make_get_nb_distinct_clusters_kernel, kmeans/kernels/utils.py:256-279. */
int32_t kmx_count_distinct_clusters(const uint32_t* labels, int32_t* seen, int32_t* result,
                                    int64_t n, int32_t k, void* stream);

/* out (m, q) = X (m, p) @ Y_t (q, p)^T.  make_matmul_2d_kernel, common/matmul.py:13-567. */
int32_t kmx_matmul(const void* X, const void* Y_t, void* out, int32_t m, int32_t p, int32_t q,
                   int32_t dtype, void* stream);

/* The scalar combined over K (multiply_fn of make_matmul_2d_kernel, common/matmul.py:64-66) and
 * the function applied to each finished sum (out_fused_elementwise_fn, :55-62), for the
 * functions the reference predefines (common/_utils.py:17-33). */
#define KMX_MATMUL_MULTIPLY 0      /* sum_k x * y: matrix cores */
#define KMX_MATMUL_MINUS 1         /* sum_k (x - y) */
#define KMX_MATMUL_PLUS 2          /* sum_k (x + y) */
#define KMX_MATMUL_OUT_IDENTITY 0
#define KMX_MATMUL_OUT_SQUARE 1    /* v * v */
#define KMX_MATMUL_OUT_DIVIDE_BY 2 /* v / out_param */

/* out[i, j] = out_op(sum_k multiply_op(X[i, k], Y_t[j, k])).  make_matmul_2d_kernel with
 * multiply_fn / out_fused_elementwise_fn, common/matmul.py:13-70,300-567. */
int32_t kmx_matmul_fused(const void* X, const void* Y_t, void* out, int32_t m, int32_t p,
                         int32_t q, int32_t multiply_op, int32_t out_op, double out_param,
                         int32_t dtype, void* stream);

/* ------------------------------------------------------------------------------------ *
 * Machine probes (benchmarks only)                                                      *
 * ------------------------------------------------------------------------------------ */

/* What this GPU reaches on the simplest kernels, so that a benchmark can price the KMeans
 * kernels against measured ceilings next to the datasheet ones: a device-to-device copy
 * (n_bytes read + n_bytes written), a read-only pass over n_bytes, and a stream of independent
 * matrix-core instructions (kind 0: v_mfma_f32_32x32x2_f32, 1: v_mfma_f32_32x32x16_f16,
 * 2: v_mfma_f64_16x16x4_f64; *flops_host receives the flops of the launch).  The caller times
 * them on `stream`.  n_bytes: a multiple of 16, pointers 16-byte aligned; scratch: 1 MiB of
 * device memory.  They have no counterpart in the reference, which publishes no roofline
 * figures (benchmark/kmeans.py only times whole fits). */
int32_t kmx_probe_copy(const void* src, void* dst, size_t n_bytes, void* stream);
int32_t kmx_probe_read(const void* src, size_t n_bytes, void* scratch, void* stream);
int32_t kmx_probe_mfma(int32_t kind, int32_t iters, void* scratch, double* flops_host, void* stream);

/* How matrix-core and vector-ALU instructions share a SIMD's issue slots: `iters` rounds of two
 * independent MFMAs (kind 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_32x32x2_f32, 2: none) and
 * 2 * valu_per_mfma (0, 8, 16 or 32) independent v_max3_f32, three waves per SIMD on every SIMD.
 * The caller times the launch; scratch: 1 MiB.  It has no counterpart in the reference
 * (benchmarks only). */
int32_t kmx_probe_issue(int32_t kind, int32_t valu_per_mfma, int32_t iters, void* scratch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_KMEANS_H */
