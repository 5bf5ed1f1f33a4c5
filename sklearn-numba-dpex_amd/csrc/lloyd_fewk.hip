// fp32 fused Lloyd step for FEW clusters (k <= 16) on WIDE samples (64 < d <= 1792), reading X
// once per iteration.
//
// Replaces, for these shapes, the kernel pair fused_lloyd_single_step
// (sklearn_numba_dpex/kmeans/kernels/lloyd_single_step.py:35-424) + the reduction of the
// privatised sums (kmeans/drivers.py:301-312); the reduction over the workgroups' partial sums
// and the finalisation stay with lloyd.hip.
//
// With few clusters neither the labels nor the sums cost much arithmetic; what costs is reading
// X twice (once for the labels, once more for the sums once the labels are known), which the
// streaming vector-ALU step does, or sorting the samples by label first, which the bucketed sums
// do.  Here a workgroup keeps a tile of S samples x all features in LDS and uses it twice:
//
//   * labels: scores(16 clusters x 16 samples) = C (16 x d) X_tile (d x 16) - 0.5||c||^2 with
//     v_mfma_f32_16x16x4_f32 (A: lane l = cluster l % 16, feature l / 16; B: lane l = feature
//     l / 16, sample l % 16; D: lane l holds clusters 4 (l / 16) + r of sample l % 16).  Each of
//     the NW waves (four; eight beyond 512 features) takes its share of the features, whose
//     centroid values it holds in registers for the whole kernel, and the partial score tiles
//     are added in wave order (strict '>' in increasing cluster order: the lowest index wins).
//   * sums: sums(16 clusters x 16 features) += M (16 clusters x 4 samples) X_tile^T (4 samples x
//     16 features), M = w_i where sample i carries the row's label and 0 elsewhere; the feature
//     row d of the tile holds ones, so column d collects the cluster sizes.  A wave owns every
//     NW-th block of 16 features and keeps their accumulators in registers until the end.
//
// The rows of the next tile travel from memory into registers while the tile in LDS is worked
// on - or, beyond 512 features with a row-major copy of X, straight into LDS, two workgroups per
// compute unit taking turns at waiting and working.  fp32 accumulation per workgroup (a few
// thousand samples); fewk_reduce_kernel adds the workgroups' partial sums and finishes the iteration.
#include "lloyd_layout.h"
#include "lloyd_tail.h"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

// Barrier between two passes over the LDS of a workgroup: the wave's own LDS accesses are done, then
// the barrier.  (__syncthreads() is a fence as well, and a fence waits for every load from memory
// into LDS that is in flight - the next tile, which is wanted only a whole tile later.)
__device__ __forceinline__ void fewk_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

struct FewkLds {
    size_t off_part, off_lab, off_w, total;
    int rows;    // features of the tile: d, the ones, and padding up to what the unrolled loops address
    int stride;  // feature-major tile: words per feature row, S + 4
    int ds;      // sample-major tile: words per sample, >= rows and = 20 mod 64
                 // (either way the lanes of a matrix operand fall on different banks, nearly)
};

// K steps of four features per wave for d features shared by nw waves
__host__ __device__ constexpr int fewk_kw(int d, int nw) { return (((d + 3) / 4) + nw - 1) / nw; }

__host__ __device__ inline FewkLds fewk_lds(int d, int S, int nw, bool two_tiles = false) {
    FewkLds s;
    const int kw = fewk_kw(d, nw);
    // the label pass of the last wave reads K steps (nw - 1) kw .. (nw - 1) kw + 8 ceil(kw / 8) - 1
    // (with zero centroid values past its share), the sums pass blocks of 16 rows up to row d
    const int rows_k = 4 * ((nw - 1) * kw + 8 * ((kw + 7) / 8));
    const int rows_f = 16 * ((d + 1 + 15) / 16);
    s.rows = rows_k > rows_f ? rows_k : rows_f;
    s.stride = S + 4;
    s.ds = s.rows + ((20 - s.rows % 64) + 64) % 64;
    // (room for the larger of the two layouts: the launch does not depend on which one runs)
    // (two_tiles: the sample-major tile twice - one is worked on while the next one arrives)
    const size_t fm = (size_t)s.rows * s.stride * 4, sm = (size_t)S * s.ds * 4 * (two_tiles ? 2 : 1);
    s.off_part = fm > sm ? fm : sm;                          // [nw waves][S / 16][16 clusters][16 samples]
    s.off_lab = s.off_part + (size_t)nw * (S / 16) * 256 * 4;
    s.off_w = s.off_lab + (size_t)S * 4;
    s.total = s.off_w + (size_t)S * 4;
    return s;
}

// 128-bit pieces of the next tile a thread holds in registers (d * S / 4 values over the threads)
constexpr int fewk_prefetch(int kw, int s_log, int nw) {
    if (nw == 8) return kw <= 26 ? 7 : kw <= 38 ? 10 : 16;
    return (kw <= 8 && s_log == 5) ? 4 : kw <= 16 ? 8 : kw <= 32 ? 10 : kw <= 52 ? 13 : 19;  // ((8, 6): 8)
}

// KW: K steps of four features per wave the kernel is unrolled for (d <= 16 KW); S_LOG: log2 of
// the samples per tile.  Row offsets inside the tile are compile-time multiples of the row stride,
// so that the reads of the unrolled loops differ by immediate offsets only.
// RM: the tile is read from the row-major copy of X, (n, d) with d a multiple of 4 - S whole
// samples are one contiguous stretch of memory, where the feature-major array gives d separate
// pieces of 4 S bytes - and kept sample-major in LDS.
// NW: waves per workgroup.  Beyond 512 features eight waves share the tile: a wave then holds half as
// many centroid values, sums and pieces of the next tile, twice as many waves fit a SIMD, and the waits
// of one wave (the tile's reads before its matrix instructions, the barriers between the passes) are
// filled by another.
// (two waves per SIMD - two workgroups of four waves per compute unit - up to 832 features: 256
// registers; four with tiles of 32 samples of up to 128 features and with eight waves up to 832)
constexpr int fewk_waves_per_simd(int kw, int s_log, int nw, int direct = 0) {
    if (nw == 8) return (direct == 1 && kw <= 26) ? 4 : 2;
    if (direct == 1) return 4;
    return (kw <= 8 && s_log == 5) ? 4 : kw <= 52 ? 2 : 1;
}

// DIRECT (with RM): a tile travels from memory straight into LDS (global_load_lds_dwordx4: the 64
// lanes of a wave fill 1024 consecutive bytes of a sample's row) instead of into registers, from
// where the waves had to store it once the tile in LDS was free: no registers are held for it, the
// reads of a pass can be in flight together, and no wave spends instructions on the copy.
//   1: one tile per workgroup; the workgroup waits for it, and the other workgroup of the compute
//      unit works meanwhile (two workgroups of eight waves, 128 registers);
//   2: two tiles, the next one arrives while this one is worked on (one workgroup per compute unit).
template <int KW, int S_LOG, bool RM, int NW, int DIRECT = 0>
__global__ __launch_bounds__(64 * NW)
__attribute__((amdgpu_waves_per_eu(fewk_waves_per_simd(KW, S_LOG, NW, DIRECT),
                                   fewk_waves_per_simd(KW, S_LOG, NW, DIRECT))))
void lloyd_fewk_kernel(
    const float* __restrict__ X_t, const float* __restrict__ X_rm, const float* __restrict__ sample_weight,
    const float* __restrict__ centroids_t, const float* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    float* __restrict__ partial, kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k, int vec_ok) {
    if (status->state != KMX_RUNNING) return;
    constexpr int FBW = KW / 4 + 1;  // blocks of 16 features per wave
    constexpr int PF = fewk_prefetch(KW, S_LOG, NW);
    constexpr int S = 1 << S_LOG, NB = S >> 4, STRIDE = S + 4;
    constexpr int NT = 64 * NW;    // threads
    constexpr int SPW = S / NW;    // samples of the tile a wave fetches
    extern __shared__ __align__(16) unsigned char smem_raw[];
    static_assert(!DIRECT || RM, "tiles arrive in LDS directly only from the row-major copy");
    const FewkLds lay = fewk_lds(d, S, NW, DIRECT == 2);
    float* tile = reinterpret_cast<float*>(smem_raw);                     // [rows][STRIDE]
    float* part = reinterpret_cast<float*>(smem_raw + lay.off_part);
    uint32_t* lab = reinterpret_cast<uint32_t*>(smem_raw + lay.off_lab);  // [S]
    float* wts = reinterpret_cast<float*>(smem_raw + lay.off_w);          // [S]
    const int rows = lay.rows;
    const int DS = lay.ds;
    __shared__ unsigned int changed_block;

    // (the wave index in a scalar register: conditions on it are then branches of the wave, not
    // masks over its lanes)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int g4 = lane >> 4, m16 = lane & 15;
    const int kw = fewk_kw(d, NW);  // K steps per wave (<= KW)
    const int ks0 = wave * kw;
    const int n_fb = (d + 1 + 15) >> 4;  // blocks of 16 features, the row of ones included
    // wave w takes the blocks w, w + NW, ...: FBW of them whatever d is, a block past the last one
    // standing for the last (its sums are not written) - no branch inside the loop over the
    // samples, around which the compiler would copy all the accumulators

    // the wave's centroid values: cluster m16, feature 4 (ks0 + s) + g4
    float ca[KW];
    // -0.5||c||^2 of the clusters 4 g4 + r: the start of wave 0's scores
    v4f start;
    // (every lane loads - a clamped address where it has no value - so that the loads are issued
    // together: under a condition each one became a block of its own that waited for its value)
    auto load_centroids = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < KW; ++s) {
            const int f = 4 * (ks0 + s) + g4;
            const bool has = s < kw && f < d && m16 < k;
            const float v = centroids_t[has ? (size_t)f * k + m16 : (size_t)0];
            ca[s] = has ? v : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float hn = half_norms[4 * g4 + r < k ? 4 * g4 + r : 0];
            start[r] = (wave == 0 && 4 * g4 + r < k) ? -hn : 0.0f;
        }
    };
    // (DIRECT: after the first tile has been asked for)
    if constexpr (!DIRECT) load_centroids();
    // past the features: ones (feature d, the cluster sizes), then zeros; never overwritten
    if (DIRECT) {
        // (both tiles, and zeros in the rows as well: the rows past the last sample are never loaded)
        for (int r = wave; r < (DIRECT == 2 ? 2 : 1) * S; r += NW)
            for (int c = lane; c < DS; c += 64) tile[r * DS + c] = c == d ? 1.0f : 0.0f;
        fewk_lds_barrier();
    } else if (RM) {
        for (int idx = threadIdx.x; idx < S * (DS - d); idx += NT) {
            const int sm = idx / (DS - d), c = idx - sm * (DS - d);
            tile[sm * DS + d + c] = c == 0 ? 1.0f : 0.0f;
        }
    } else {
        for (int idx = threadIdx.x; idx < (rows - d) * STRIDE; idx += NT)
            tile[d * STRIDE + idx] = idx < STRIDE ? 1.0f : 0.0f;
    }
    if (threadIdx.x == 0) changed_block = 0;

    v4f acc[FBW];
#pragma unroll
    for (int i = 0; i < FBW; ++i) acc[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    unsigned int changed = 0;

    // The tile as 128-bit pieces, PF per thread.
    // Feature-major: the thread's piece u is four samples (its quarter q_t of the row... of S / 4)
    // of feature f_t + u * RSTEP.
    // Row-major: the S / NW samples of a wave are one contiguous stretch of (S / NW) d floats; lane l
    // takes its pieces l, l + 64, ...; piece i holds features 4 (i % P) .. + 3 of sample i / P,
    // P = d / 4.
    constexpr int Q_LOG = S_LOG - 2, RSTEP = NT >> Q_LOG;
    const int f_t = threadIdx.x >> Q_LOG, q_t = threadIdx.x & ((1 << Q_LOG) - 1);
    const size_t x_mine = (size_t)f_t * n + 4 * q_t;  // (the rest of an address is the same for all threads)
    float* const tile_mine = tile + f_t * STRIDE + 4 * q_t;
    const int P = d >> 2, wave_pieces = SPW * P;
    float4 pf[PF];
    // (and, every fourth thread, the weight and the previous label of one sample)
    float w_next = 0.0f;
    uint32_t pl_next = 0u;
    auto fetch = [&](const int64_t s0) __attribute__((always_inline)) {
        const bool whole = vec_ok && s0 + S <= n;  // workgroup-uniform
        if ((int)threadIdx.x < 4 * S && (threadIdx.x & 3) == 0 && s0 + (threadIdx.x >> 2) < n) {
            w_next = sample_weight[s0 + (threadIdx.x >> 2)];
            pl_next = labels_prev[s0 + (threadIdx.x >> 2)];
        }
        if constexpr (RM) {
            // (pieces of samples past the end are not read)
            const int64_t left = n - (s0 + (int64_t)wave * SPW);  // samples of the wave's stretch that exist
            const int64_t live_pieces = left <= 0 ? 0 : (left >= SPW ? wave_pieces : left * P);
            const float4* src = reinterpret_cast<const float4*>(X_rm + (size_t)(s0 + wave * SPW) * d);
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                const int i = lane + 64 * u;
                pf[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (i < live_pieces) pf[u] = src[i];
            }
        } else {
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                pf[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (f_t + u * RSTEP < d) {
                    const float* p = X_t + ((size_t)(u * RSTEP) * n + s0) + x_mine;
                    if (whole) {
                        pf[u] = *reinterpret_cast<const float4*>(p);
                    } else {
                        const int64_t i = s0 + 4 * q_t;
                        if (i < n) pf[u].x = p[0];
                        if (i + 1 < n) pf[u].y = p[1];
                        if (i + 2 < n) pf[u].z = p[2];
                        if (i + 3 < n) pf[u].w = p[3];
                    }
                }
            }
        }
    };
    auto deposit = [&]() __attribute__((always_inline)) {
        if constexpr (RM) {
            // (sample, piece inside the sample) of the lane's pieces, stepped from one to the next;
            // the start is made opaque so that the chain is recomputed per tile instead of
            // occupying a register per piece for the whole kernel
            int sm = lane / P, r = lane - sm * P;
            asm volatile("" : "+v"(sm), "+v"(r));
            const int step_s = 64 / P, step_r = 64 - step_s * P;
#pragma unroll
            for (int u = 0; u < PF; ++u) {
                if (lane + 64 * u < wave_pieces)
                    *reinterpret_cast<float4*>(tile + (wave * SPW + sm) * DS + 4 * r) = pf[u];
                sm += step_s;
                r += step_r;
                if (r >= P) {
                    r -= P;
                    sm += 1;
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < PF; ++u)
                if (f_t + u * RSTEP < d) *reinterpret_cast<float4*>(tile_mine + u * RSTEP * STRIDE) = pf[u];
        }
    };

    // DIRECT: the wave's SPW rows of the tile at s0, 64 pieces per instruction, into the tile at word
    // offset buf of the LDS (weight and previous label travel in registers as above)
    constexpr int PC = (KW * NW + 63) / 64;  // instructions per row for the widest sample of this kernel
    const int full_chunks = P >> 6, last_chunk = P & 63;  // instructions of 64 pieces per row, pieces of one more
    auto issue = [&](const int64_t s0, const int buf) __attribute__((always_inline)) {
        // (the thread that will write the sample's label holds its weight and previous label)
        if ((int)threadIdx.x < 16 * S && (threadIdx.x & 15) == 0 && s0 + (threadIdx.x >> 4) < n) {
            w_next = sample_weight[s0 + (threadIdx.x >> 4)];
            pl_next = labels_prev[s0 + (threadIdx.x >> 4)];
        }
#pragma unroll
        for (int rr = 0; rr < SPW; ++rr) {
            const int row = wave * SPW + rr;
            if (s0 + row < n) {  // wave-uniform
                const float* src = X_rm + (size_t)(s0 + row) * d + 4 * lane;
                float* dst = tile + buf + row * DS;
#pragma unroll
                for (int c = 0; c < PC; ++c) {
                    if (c < full_chunks) {  // wave-uniform
                        __builtin_amdgcn_global_load_lds(
                            (const __attribute__((address_space(1))) void*)(src + 256 * c),
                            (__attribute__((address_space(3))) void*)(dst + 256 * c), 16, 0, 0);
                    } else if (c == full_chunks && lane < last_chunk) {
                        __builtin_amdgcn_global_load_lds(
                            (const __attribute__((address_space(1))) void*)(src + 256 * c),
                            (__attribute__((address_space(3))) void*)(dst + 256 * c), 16, 0, 0);
                    }
                }
            }
        }
    };

    const int64_t n_tiles = (n + S - 1) >> S_LOG;
    int64_t t = blockIdx.x;
    const int tile_words = S * DS;
    int cur = 0;  // DIRECT: word offset of the tile that is worked on
    if (t < n_tiles) {
        if constexpr (DIRECT)
            issue(t << S_LOG, 0);
        else
            fetch(t << S_LOG);
    }
    if constexpr (DIRECT) load_centroids();
    // the wave's first row of the label pass (lane: feature g4 of a K step, sample m16 of a block)
    // and of the sums pass (lane: feature m16 of a block of 16, sample g4 of a group of four)
    const float* const col_labels0 = RM ? tile + m16 * DS + 4 * ks0 + g4 : tile + (4 * ks0 + g4) * STRIDE + m16;
    // (the wave's blocks w, w + NW, ... lie FB_STEP words apart: one address register per SUMS_G blocks,
    // the rest of an address is an immediate offset - a register per block, each stepped through the
    // tile, left the compiler no registers to keep the reads of a group in flight together, and every
    // matrix instruction waited for a read of its own.  A block past the last one reads whatever lies
    // there, inside the tile or behind it; its sums are not used.)
    constexpr int FB_STEP = RM ? 16 * NW : 16 * NW * STRIDE;
    constexpr int SUMS_G = (15000 / FB_STEP) < FBW ? (15000 / FB_STEP) : FBW;
    constexpr int SUMS_NBASE = (FBW + SUMS_G - 1) / SUMS_G;
    const float* const col_sums00 = RM ? tile + g4 * DS + 16 * wave + m16 : tile + (16 * wave + m16) * STRIDE + g4;
    (void)n_fb;
    for (; t < n_tiles; t += gridDim.x) {
        const int64_t s0 = t << S_LOG;
        float w_mine;
        uint32_t pl_mine;
        if constexpr (DIRECT) {
            // the tile has arrived (every wave waits for its own rows, then for the others), and the
            // other tile is no longer read
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            w_mine = w_next;
            pl_mine = pl_next;
            if constexpr (DIRECT == 2)
                if (t + gridDim.x < n_tiles) issue((t + gridDim.x) << S_LOG, tile_words - cur);
        } else {
            __syncthreads();  // the tile before this one is no longer read
            deposit();
            w_mine = w_next;
            pl_mine = pl_next;
            if (t + gridDim.x < n_tiles) fetch((t + gridDim.x) << S_LOG);
            __syncthreads();
        }
        const float* const col_labels = col_labels0 + cur;
        const float* const col_sums0 = col_sums00 + cur;

        // labels: partial scores of the wave's quarter of the features, eight K steps at a time
        // (their reads of the tile, for all sample blocks, in flight together), two chains of
        // accumulation per sample block
        {
            v4f sc0[NB], sc1[NB];
#pragma unroll
            for (int sb = 0; sb < NB; ++sb) {
                sc0[sb] = start;
                sc1[sb] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            }
#pragma unroll
            for (int c0 = 0; c0 < KW; c0 += 8) {
                if (c0 < kw) {  // wave-uniform
                    float b[NB][8];
                    // (past the wave's share the centroid value is zero and the rows exist)
#pragma unroll
                    for (int sb = 0; sb < NB; ++sb)
#pragma unroll
                        for (int j = 0; j < 8; ++j)
                            b[sb][j] = RM ? col_labels[16 * sb * DS + 4 * (c0 + j)]
                                          : col_labels[4 * (c0 + j) * STRIDE + 16 * sb];
                    // (the reads stay above this line: left alone, the compiler moves each one down to
                    // the matrix instruction that uses it, which then waits a full trip to the LDS)
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int j = 0; j < 8; j += 2)
#pragma unroll
                        for (int sb = 0; sb < NB; ++sb) {
                            if (c0 + j < KW)
                                sc0[sb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j < KW ? c0 + j : 0], b[sb][j],
                                                                               sc0[sb], 0, 0, 0);
                            if (c0 + j + 1 < KW)
                                sc1[sb] = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j + 1 < KW ? c0 + j + 1 : 0],
                                                                               b[sb][j + 1], sc1[sb], 0, 0, 0);
                        }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (DIRECT) {
                // [wave][sample][cluster]: the lane's four clusters are one 128-bit store
                static_assert(!DIRECT || NB == 1, "one block of 16 samples per tile");
                *reinterpret_cast<v4f*>(part + (wave << 8) + (m16 << 4) + 4 * g4) = sc0[0] + sc1[0];
            } else {
#pragma unroll
                for (int sb = 0; sb < NB; ++sb) {
                    float* out = part + ((wave * NB + sb) << 8) + m16;
#pragma unroll
                    for (int r = 0; r < 4; ++r) out[(4 * g4 + r) << 4] = sc0[sb][r] + sc1[sb][r];
                }
            }
        }
        if constexpr (DIRECT)
            fewk_lds_barrier();
        else
            __syncthreads();
        // arg-max: four threads per sample, thread q on the clusters q, q + 4, ... (the four partial
        // tiles added in wave order, strict '>' in increasing cluster order), then the four combine:
        // the largest score, the lowest index among equals
        if constexpr (DIRECT) {
            // sixteen threads per sample, one per cluster: the partial scores of the waves added in
            // wave order, then the largest score, the lowest index among equals (a score that does not
            // compare, or a cluster past the last, never wins)
            if ((int)threadIdx.x < 16 * S) {
                const int m = threadIdx.x >> 4, c = threadIdx.x & 15;
                float best = part[threadIdx.x];
#pragma unroll
                for (int wv = 1; wv < NW; ++wv) best += part[(wv << 8) + threadIdx.x];
                uint32_t bi = (uint32_t)c;
                if (!(c < k && best > -kmx_inf<float>())) {
                    best = -kmx_inf<float>();
                    bi = 0xffffffffu;
                }
#pragma unroll
                for (int off = 1; off <= 8; off <<= 1) {
                    const float ov = __shfl_xor(best, off, 64);
                    const uint32_t oi = __shfl_xor(bi, off, 64);
                    const bool take = ov > best || (ov == best && oi < bi);
                    best = take ? ov : best;
                    bi = take ? oi : bi;
                }
                if (bi == 0xffffffffu) bi = 0u;  // no score compares: the reference's running arg-min keeps 0
                const int64_t gi = s0 + m;
                const bool live = gi < n;
                if (c == 0) {
                    lab[m] = bi;
                    wts[m] = live ? w_mine : 0.0f;
                    if (live) {
                        labels[gi] = bi;
                        changed += pl_mine != bi ? 1u : 0u;
                    }
                }
            }
        } else if ((int)threadIdx.x < 4 * S) {
            const int s = threadIdx.x >> 2, q = threadIdx.x & 3, sb = s >> 4, m = s & 15;
            float best = -kmx_inf<float>();
            uint32_t bi = 0xffffffffu;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = q + 4 * j;
                if (c < k) {
                    float v = part[((0 * NB + sb) << 8) + (c << 4) + m];
#pragma unroll
                    for (int wv = 1; wv < NW; ++wv) v += part[((wv * NB + sb) << 8) + (c << 4) + m];
                    if (v > best) {
                        best = v;
                        bi = (uint32_t)c;
                    }
                }
            }
#pragma unroll
            for (int off = 1; off <= 2; off <<= 1) {
                const float ov = __shfl_xor(best, off, 64);
                const uint32_t oi = __shfl_xor(bi, off, 64);
                if (ov > best || (ov == best && oi < bi)) {
                    best = ov;
                    bi = oi;
                }
            }
            if (bi == 0xffffffffu) bi = 0u;  // no score compares: the reference's running arg-min keeps 0
            const int64_t gi = s0 + s;
            const bool live = gi < n;
            if (q == 0) {
                lab[s] = bi;
                wts[s] = live ? w_mine : 0.0f;
                if (live) {
                    labels[gi] = bi;
                    changed += pl_mine != bi ? 1u : 0u;
                }
            }
        }
        if constexpr (DIRECT)
            fewk_lds_barrier();
        else
            __syncthreads();

        // sums: the wave's feature blocks, four samples per matrix instruction
        // (U groups of four samples at a time, their reads in flight together; the loop is kept a
        // loop: unrolled, its S / 4 addresses would each take a register for the whole kernel)
        constexpr int U = DIRECT ? (FBW <= 7 ? 4 : 2) : FBW <= 5 ? 4 : FBW <= 9 ? 2 : 1;
        int at = 0;  // offset of the group of samples inside a column of the tile
        const int at_step = RM ? 4 * U * DS : 4 * U;
#pragma unroll 1
        for (int sc4 = 0; sc4 < (S >> 2); sc4 += U) {
            float aw[U], b[U][FBW];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int s = 4 * (sc4 + u) + g4;
                const uint32_t lb = lab[s];
                const float wv = wts[s];
                aw[u] = lb == (uint32_t)m16 ? wv : 0.0f;
#pragma unroll
                for (int g = 0; g < SUMS_NBASE; ++g) {
                    const float* base = col_sums0 + g * SUMS_G * FB_STEP + at + (RM ? 4 * u * DS : 4 * u);
#pragma unroll
                    for (int i = g * SUMS_G; i < (g + 1) * SUMS_G && i < FBW; ++i) b[u][i] = base[(i - g * SUMS_G) * FB_STEP];
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // (all reads of the groups, then their matrix instructions)
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < FBW; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[u], b[u][i], acc[i], 0, 0, 0);
            at += at_step;
        }
        if constexpr (DIRECT == 2) cur = tile_words - cur;
        if constexpr (DIRECT == 1) {
            // (the tile is no longer read: the next one may arrive)
            if (t + gridDim.x < n_tiles) {
                fewk_lds_barrier();
                issue((t + gridDim.x) << S_LOG, 0);
            }
        }
    }

    // The workgroup's sums as they lie in the registers: slot ((wave FBW + i) 4 + r) 64 + lane of
    // the workgroup's stretch of `partial` (whole cache lines per store; fewk_reduce_kernel knows
    // which cluster and feature a slot stands for).
    float* out = partial + (size_t)blockIdx.x * (NW * FBW * 256) + (size_t)wave * (FBW * 256) + lane;
    // (the rows of clusters past the last one are neither written nor read)
#pragma unroll
    for (int i = 0; i < FBW; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (4 * g4 + r < k) out[(i * 4 + r) * 64] = acc[i][r];
    if (changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
}

// Up to 128 features with a row-major copy of X: every WAVE works on tiles of 16 samples of its
// own, with no barrier and no exchange between waves - at this width a workgroup's tile is so small
// that the barriers and the bookkeeping around it (some 400 instructions per wave and tile for 40
// matrix instructions) cost more than the arithmetic.  The wave holds the centroid values of all
// features in registers (KS K steps of four), its scores are complete in its own registers (the
// arg-max is three compares and two exchanges between the lane groups), and it keeps the sums of
// all NFB feature blocks.  At the end the four waves of a workgroup add their sums in wave order.
constexpr int fewk_wave_ds(int cols) { return cols + ((20 - cols % 64) + 64) % 64; }
__host__ __device__ constexpr int fewk_wave_cols(int d, int nfb) {
    return 4 * ((d + 3) / 4) > 16 * nfb ? 4 * ((d + 3) / 4) : 16 * nfb;
}
template <int KS, int NFB>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) void lloyd_fewk_wave_kernel(
    const float* __restrict__ X_rm, const float* __restrict__ sample_weight,
    const float* __restrict__ centroids_t, const float* __restrict__ half_norms,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    float* __restrict__ partial, kmx_lloyd_status* __restrict__ status, int64_t n, int d, int k) {
    if (status->state != KMX_RUNNING) return;
    constexpr int PF = (16 * 16 * NFB / 4 + 63) / 64;  // 128-bit pieces per lane of a tile of 16 samples
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int g4 = lane >> 4, m16 = lane & 15;
    const int DS = fewk_wave_ds(fewk_wave_cols(d, NFB));
    float* tile = reinterpret_cast<float*>(smem_raw) + wave * 16 * DS;  // [16 samples][DS], the wave's own
    const int ksteps = (d + 3) >> 2;
    const int n_fb = (d + 1 + 15) >> 4;
    __shared__ unsigned int changed_block;

    // (every lane loads, from a clamped address where it has no value: the loads are issued together)
    float ca[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int f = 4 * s + g4;
        const bool has = f < d && m16 < k;
        const float v = centroids_t[has ? (size_t)f * k + m16 : (size_t)0];
        ca[s] = has ? v : 0.0f;
    }
    v4f start;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const float hn = half_norms[4 * g4 + r < k ? 4 * g4 + r : 0];
        start[r] = (4 * g4 + r < k) ? -hn : 0.0f;
    }
    // past the features: ones (feature d, the cluster sizes), then zeros; never overwritten
    for (int idx = lane; idx < 16 * (DS - d); idx += 64) {
        const int sm = idx / (DS - d), c = idx - sm * (DS - d);
        tile[sm * DS + d + c] = c == 0 ? 1.0f : 0.0f;
    }
    if (threadIdx.x == 0) changed_block = 0;
    __syncthreads();

    v4f acc[NFB];
#pragma unroll
    for (int i = 0; i < NFB; ++i) acc[i] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    unsigned int changed = 0;

    // a tile is one contiguous stretch of 16 d floats; lane l takes its 128-bit pieces l, l + 64, ...;
    // piece i holds features 4 (i % P) .. + 3 of sample i / P, P = d / 4
    const int P = d >> 2, tile_pieces = 16 * P;
    float4 pf[PF];
    float w_next = 0.0f;
    uint32_t pl_next = 0u;
    auto fetch = [&](const int64_t s0) __attribute__((always_inline)) {
        if (g4 == 0 && s0 + m16 < n) {
            w_next = sample_weight[s0 + m16];
            pl_next = labels_prev[s0 + m16];
        }
        const int64_t left = n - s0;
        const int live_pieces = left >= 16 ? tile_pieces : (int)left * P;
        const float4* src = reinterpret_cast<const float4*>(X_rm + (size_t)s0 * d);
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            const int i = lane + 64 * u;
            pf[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (i < live_pieces) pf[u] = src[i];
        }
    };
    auto deposit = [&]() __attribute__((always_inline)) {
        int sm = lane / P, r = lane - sm * P;
        asm volatile("" : "+v"(sm), "+v"(r));  // (recomputed per tile instead of a register per piece)
        const int step_s = 64 / P, step_r = 64 - step_s * P;
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            if (lane + 64 * u < tile_pieces) *reinterpret_cast<float4*>(tile + sm * DS + 4 * r) = pf[u];
            sm += step_s;
            r += step_r;
            if (r >= P) {
                r -= P;
                sm += 1;
            }
        }
    };

    const int64_t n_tiles = (n + 15) >> 4;
    const int64_t t_step = (int64_t)gridDim.x * 4;
    int64_t t = (int64_t)blockIdx.x * 4 + wave;
    if (t < n_tiles) fetch(t << 4);
    const float* const col_labels = tile + m16 * DS + g4;       // feature g4 of a K step, sample m16
    const float* const col_sums = tile + g4 * DS + m16;         // sample g4 of a group of four, feature m16 of a block
    for (; t < n_tiles; t += t_step) {
        const int64_t s0 = t << 4;
        deposit();
        const float w_mine = w_next;
        const uint32_t pl_mine = pl_next;
        if (t + t_step < n_tiles) fetch((t + t_step) << 4);

        // labels: all K steps, two chains of accumulation
        v4f sc0 = start, sc1 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c0 = 0; c0 < KS; c0 += 8) {
            if (c0 < ksteps) {  // wave-uniform (past d the centroid values are zero and the columns exist)
                float b[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) b[j] = col_labels[4 * (c0 + j < KS ? c0 + j : KS - 1)];
                // (the reads stay above this line: left alone, the compiler moves each one down to the
                // matrix instruction that uses it, which then waits a full trip to the LDS)
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    if (c0 + j < KS) sc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j < KS ? c0 + j : 0], b[j], sc0, 0, 0, 0);
                    if (c0 + j + 1 < KS)
                        sc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j + 1 < KS ? c0 + j + 1 : 0], b[j + 1], sc1, 0,
                                                                   0, 0);
                }
            }
        }
        // arg-max of sample m16: the lane's clusters 4 g4 + r in increasing order (strict '>'), then
        // the four lane groups: the largest score, the lowest index among equals
        float best = -kmx_inf<float>();
        uint32_t bi = 0xffffffffu;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = sc0[r] + sc1[r];
            if (4 * g4 + r < k && v > best) {
                best = v;
                bi = (uint32_t)(4 * g4 + r);
            }
        }
#pragma unroll
        for (int off = 16; off <= 32; off <<= 1) {
            const float ov = __shfl_xor(best, off, 64);
            const uint32_t oi = __shfl_xor(bi, off, 64);
            const bool take = ov > best || (ov == best && oi < bi);
            best = take ? ov : best;
            bi = take ? oi : bi;
        }
        if (bi == 0xffffffffu) bi = 0u;  // no score compares: the reference's running arg-min keeps 0
        const bool live = s0 + m16 < n;
        if (g4 == 0 && live) {
            labels[s0 + m16] = bi;
            changed += pl_mine != bi ? 1u : 0u;
        }
        // (lanes 0 .. 15 hold label and weight of sample m16)
        const float w_lane = live ? w_mine : 0.0f;

        // sums: four samples per matrix instruction; the row of sample 4 c + g4 carries its weight
        // in the column of its cluster (two groups of four samples at a time: their reads, then
        // their matrix instructions)
#pragma unroll
        for (int c0 = 0; c0 < 4; c0 += 2) {
            float aw[2], b[2][NFB];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int c = c0 + u;
                const uint32_t lb = __shfl(bi, 4 * c + g4, 64);
                const float wv = __shfl(w_lane, 4 * c + g4, 64);
                aw[u] = lb == (uint32_t)m16 ? wv : 0.0f;
#pragma unroll
                for (int i = 0; i < NFB; ++i) b[u][i] = col_sums[4 * c * DS + 16 * i];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < NFB; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(aw[u], b[u][i], acc[i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    // the four waves' sums are added in wave order (through the LDS of the tiles, now free): one
    // partial per workgroup, slot (fb 4 + r) 64 + lane
    if (changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    float* mine = reinterpret_cast<float*>(smem_raw) + wave * (NFB * 256) + lane;  // (NFB * 256 <= 16 DS)
#pragma unroll
    for (int i = 0; i < NFB; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) mine[(i * 4 + r) * 64] = acc[i][r];
    __syncthreads();
    const float* all = reinterpret_cast<const float*>(smem_raw);
    float* out = partial + (size_t)blockIdx.x * (NFB * 256);
    for (int slot = threadIdx.x; slot < NFB * 256; slot += 256)
        out[slot] = ((all[slot] + all[NFB * 256 + slot]) + all[2 * NFB * 256 + slot]) + all[3 * NFB * 256 + slot];
    (void)n_fb;
    if (threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
}

// Sum of the workgroups' partial sums, slot by slot and always in the same order, then the end of
// the iteration.  A workgroup takes 32 slots; its 1024 threads are 32 groups that each add every
// 32nd partial (sixteen loads in flight), and the groups are added in order.  The totals go
// into the 64-bit fixed-point sums of the run, (d + 1, k) feature-major with the sizes in row d,
// by device-scope stores, and the workgroup that gets done last finishes the iteration - empty
// clusters, division, shift, convergence test, what the next step needs - reading them with
// device-scope loads: one launch instead of two.
// PER_WAVE: the partials are those of lloyd_fewk_wave_kernel - FBW blocks of 16 features each,
// block fb in slots 256 fb .. 256 fb + 255.
template <int FBW, bool PER_WAVE, int NW>
__global__ __launch_bounds__(1024) void fewk_reduce_kernel(const float* __restrict__ partial, int n_partials,
                                                          unsigned long long* __restrict__ gsum,
                                                          const int* __restrict__ q_exp, int d, int k,
                                                          const LloydTail<float> tail) {
    extern __shared__ __align__(16) unsigned char red_raw[];
    kmx_lloyd_status* status = tail.status;
    if (status->state != KMX_RUNNING) return;
    constexpr int NSLOT = (PER_WAVE ? 1 : NW) * FBW * 256;
    constexpr int GROUPS = 32;
    __shared__ float group_sum[GROUPS][32];
    const int sl = threadIdx.x & 31, pg = threadIdx.x >> 5;
    const int slot = blockIdx.x * 32 + sl;
    float total = 0.0f;
    // (slot -> cluster: lane group and register of the step's accumulators; clusters past the last
    // one were not written)
    const bool used = slot < NSLOT && 4 * ((slot & 63) >> 4) + ((slot >> 6) & 3) < k;
    if (used) {
        const float* src = partial + slot;
        int p = pg;
        for (; p + GROUPS * 15 < n_partials; p += GROUPS * 16) {
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = src[(size_t)(p + GROUPS * u) * NSLOT];
#pragma unroll
            for (int u = 0; u < 16; ++u) total += v[u];
        }
        {
            // (the rest, its loads issued together as well)
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) v[u] = p + GROUPS * u < n_partials ? src[(size_t)(p + GROUPS * u) * NSLOT] : 0.0f;
#pragma unroll
            for (int u = 0; u < 16; ++u) total += v[u];
        }
    }
    group_sum[pg][sl] = total;
    __syncthreads();
    if (threadIdx.x < 32 && used) {
        float v = group_sum[0][sl];
#pragma unroll
        for (int g = 1; g < GROUPS; ++g) v += group_sum[g][sl];
        // slot -> (feature, cluster): wave-of-the-step, block, register, lane
        const int lane = slot & 63, r = (slot >> 6) & 3, wi = slot >> 8;  // wi = wave FBW + i
        const int wave = wi / FBW, i = wi - wave * FBW;
        const int fb = PER_WAVE ? wi : wave + NW * i;
        const int f = 16 * fb + (lane & 15), c = 4 * (lane >> 4) + r;
        if (f <= d && c < k && fb < ((d + 1 + 15) >> 4))
            __hip_atomic_store(gsum + (size_t)f * k + c, (unsigned long long)__double2ll_rn(ldexp((double)v, q_exp[f])),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __shared__ unsigned int is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) is_last = (atomicAdd(&status->ticket, 1u) == gridDim.x - 1) ? 1u : 0u;
    __syncthreads();
    if (is_last != 0u) {
        lloyd_small_finalize_body<float, true, true, true>(gsum, q_exp, tail, reinterpret_cast<float*>(red_raw));
        if (threadIdx.x == 0) status->ticket = 0u;
    }
}

// Labels only (kmx_assign_labels: predict, and the last step of a fit), straight from the
// feature-major array, with no tile in LDS: for the labels alone the samples are only ever the N
// side of the products, so a lane's 64- or 128-bit load of SV consecutive samples of one feature IS
// the B operand of SV matrix instructions - sample block e of a tile holds the samples s0 + SV m + e,
// m = 0 .. 15 - and the 16 lanes of a feature read one contiguous stretch.  Eight waves share the K
// steps of a tile of 16 SV samples (centroid values in registers, as in the step above); their
// partial scores meet in LDS and sixteen threads per sample take the arg-max.
// (beyond 832 features the centroid values of a wave leave room for one workgroup per compute unit only)
constexpr int fewk_labels_waves_per_simd(int kw) { return kw <= 26 ? 4 : 2; }
template <int KW, int SV>
__global__ __launch_bounds__(512)
__attribute__((amdgpu_waves_per_eu(fewk_labels_waves_per_simd(KW), fewk_labels_waves_per_simd(KW))))
void fewk_labels_kernel(
    const float* __restrict__ X_t, const float* __restrict__ centroids_t, const float* __restrict__ half_norms,
    uint32_t* __restrict__ labels, int64_t n, int d, int k, int vec_ok) {
    constexpr int NW = 8, TS = 16 * SV;  // waves, samples per tile
    constexpr int CH = SV == 4 ? 4 : 8;   // K steps whose loads are in flight together
    __shared__ __align__(16) float part[NW][SV][256];  // [wave][block][sample m][cluster]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int g4 = lane >> 4, m16 = lane & 15;
    const int kw = fewk_kw(d, NW);  // K steps per wave (<= KW)
    const int ks0 = wave * kw;
    float ca[KW];
#pragma unroll
    for (int s = 0; s < KW; ++s) {
        const int f = 4 * (ks0 + s) + g4;
        const bool has = s < kw && f < d && m16 < k;
        const float v = centroids_t[has ? (size_t)f * k + m16 : (size_t)0];
        ca[s] = has ? v : 0.0f;
    }
    v4f start;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const float hn = half_norms[4 * g4 + r < k ? 4 * g4 + r : 0];
        start[r] = (wave == 0 && 4 * g4 + r < k) ? -hn : 0.0f;
    }
    const int64_t n_tiles = (n + TS - 1) / TS;
    for (int64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
        const int64_t s0 = t * TS;
        const bool whole = vec_ok && s0 + TS <= n;  // workgroup-uniform
        v4f sc[SV];
#pragma unroll
        for (int e = 0; e < SV; ++e) sc[e] = start;
#pragma unroll
        for (int c0 = 0; c0 < KW; c0 += CH) {
            if (c0 < kw) {  // wave-uniform (past the wave's share the centroid value is zero)
                float b[CH][SV];
#pragma unroll
                for (int j = 0; j < CH; ++j) {
                    const int s = c0 + j;
                    // (a feature past the last one: the row of the last, times a zero centroid value)
                    const int f = 4 * (ks0 + s) + g4 < d ? 4 * (ks0 + s) + g4 : d - 1;
                    const float* p = X_t + (size_t)f * n + s0 + SV * m16;
                    if (s < KW) {
                        if (whole) {
                            if constexpr (SV == 4) {
                                const float4 v = *reinterpret_cast<const float4*>(p);
                                b[j][0] = v.x; b[j][1] = v.y; b[j][2] = v.z; b[j][3] = v.w;
                            } else {
                                const float2 v = *reinterpret_cast<const float2*>(p);
                                b[j][0] = v.x; b[j][1] = v.y;
                            }
                        } else {
#pragma unroll
                            for (int e = 0; e < SV; ++e) b[j][e] = s0 + SV * m16 + e < n ? p[e] : 0.0f;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // (the loads of the chunk, then its matrix instructions)
#pragma unroll
                for (int j = 0; j < CH; ++j)
                    if (c0 + j < KW)
#pragma unroll
                        for (int e = 0; e < SV; ++e)
                            sc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j < KW ? c0 + j : 0], b[j][e], sc[e], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int e = 0; e < SV; ++e) *reinterpret_cast<v4f*>(&part[wave][e][(m16 << 4) + 4 * g4]) = sc[e];
        __syncthreads();
        // sixteen threads per sample, one per cluster: the partial scores of the waves added in wave
        // order, then the largest score, the lowest index among equals (a score that does not compare,
        // or a cluster past the last, never wins)
#pragma unroll
        for (int rep = 0; rep < (SV * 256) / 512; ++rep) {
            const int pair = threadIdx.x + 512 * rep;  // block e, sample m, cluster c
            const int e = pair >> 8, m = (pair >> 4) & 15, c = pair & 15;
            float best = part[0][e][pair & 255];
#pragma unroll
            for (int wv = 1; wv < NW; ++wv) best += part[wv][e][pair & 255];
            uint32_t bi = (uint32_t)c;
            if (!(c < k && best > -kmx_inf<float>())) {
                best = -kmx_inf<float>();
                bi = 0xffffffffu;
            }
#pragma unroll
            for (int off = 1; off <= 8; off <<= 1) {
                const float ov = __shfl_xor(best, off, 64);
                const uint32_t oi = __shfl_xor(bi, off, 64);
                const bool take = ov > best || (ov == best && oi < bi);
                best = take ? ov : best;
                bi = take ? oi : bi;
            }
            if (bi == 0xffffffffu) bi = 0u;  // no score compares: the reference's running arg-min keeps 0
            const int64_t gi = s0 + SV * m + e;
            if (c == 0 && gi < n) labels[gi] = bi;
        }
        __syncthreads();  // the partial scores are read: the next tile may overwrite them
    }
}

// The same up to 128 features, where a wave holds the centroid values of all features: every wave
// on tiles of 64 samples of its own, scores complete in its registers - no LDS, no barrier.
template <int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void fewk_labels_wave_kernel(
    const float* __restrict__ X_t, const float* __restrict__ centroids_t, const float* __restrict__ half_norms,
    uint32_t* __restrict__ labels, int64_t n, int d, int k, int vec_ok) {
    constexpr int SV = 4, TS = 16 * SV, CH = 4;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int g4 = lane >> 4, m16 = lane & 15;
    const int ksteps = (d + 3) >> 2;
    float ca[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int f = 4 * s + g4;
        const bool has = f < d && m16 < k;
        const float v = centroids_t[has ? (size_t)f * k + m16 : (size_t)0];
        ca[s] = has ? v : 0.0f;
    }
    v4f start;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const float hn = half_norms[4 * g4 + r < k ? 4 * g4 + r : 0];
        start[r] = (4 * g4 + r < k) ? -hn : 0.0f;
    }
    const int64_t n_tiles = (n + TS - 1) / TS;
    for (int64_t t = (int64_t)blockIdx.x * 4 + wave; t < n_tiles; t += (int64_t)gridDim.x * 4) {
        const int64_t s0 = t * TS;
        const bool whole = vec_ok && s0 + TS <= n;  // wave-uniform
        v4f sc[SV];
#pragma unroll
        for (int e = 0; e < SV; ++e) sc[e] = start;
#pragma unroll
        for (int c0 = 0; c0 < KS; c0 += CH) {
            if (c0 < ksteps) {  // wave-uniform (past d the centroid values are zero)
                float b[CH][SV];
#pragma unroll
                for (int j = 0; j < CH; ++j) {
                    const int f = 4 * (c0 + j) + g4 < d ? 4 * (c0 + j) + g4 : d - 1;
                    const float* p = X_t + (size_t)f * n + s0 + SV * m16;
                    if (whole) {
                        const float4 v = *reinterpret_cast<const float4*>(p);
                        b[j][0] = v.x; b[j][1] = v.y; b[j][2] = v.z; b[j][3] = v.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < SV; ++e) b[j][e] = s0 + SV * m16 + e < n ? p[e] : 0.0f;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // (the loads of the chunk, then its matrix instructions)
#pragma unroll
                for (int j = 0; j < CH; ++j)
                    if (c0 + j < KS)
#pragma unroll
                        for (int e = 0; e < SV; ++e)
                            sc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[c0 + j < KS ? c0 + j : 0], b[j][e], sc[e], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // arg-max of sample SV m16 + e: the lane's clusters 4 g4 + r in increasing order (strict '>'),
        // then the four lane groups: the largest score, the lowest index among equals
        uint32_t lab[SV];
#pragma unroll
        for (int e = 0; e < SV; ++e) {
            float best = -kmx_inf<float>();
            uint32_t bi = 0xffffffffu;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = sc[e][r];
                if (4 * g4 + r < k && v > best) {
                    best = v;
                    bi = (uint32_t)(4 * g4 + r);
                }
            }
#pragma unroll
            for (int off = 16; off <= 32; off <<= 1) {
                const float ov = __shfl_xor(best, off, 64);
                const uint32_t oi = __shfl_xor(bi, off, 64);
                const bool take = ov > best || (ov == best && oi < bi);
                best = take ? ov : best;
                bi = take ? oi : bi;
            }
            lab[e] = bi == 0xffffffffu ? 0u : bi;  // no score compares: the reference's running arg-min keeps 0
        }
        if (g4 == 0) {
            const int64_t gi = s0 + SV * m16;
            if (whole) {
                *reinterpret_cast<uint4*>(labels + gi) = make_uint4(lab[0], lab[1], lab[2], lab[3]);
            } else {
#pragma unroll
                for (int e = 0; e < SV; ++e)
                    if (gi + e < n) labels[gi + e] = lab[e];
            }
        }
    }
}

// Samples per tile (a power of two, 16 .. 64) and workgroups per compute unit.
struct FewkShape {
    int s_log, kw, nw, per_cu;
    size_t lds;
};

bool fewk_shape(int d, int k, FewkShape* out) {
    if (d <= 64 || d > 1792 || k < 1 || k > 16) return false;
    // (eight waves per workgroup beyond 512 features)
    const int nw = d > 512 ? 8 : 4;
    const int kw = fewk_kw(d, nw);
    const int kw_t = nw == 8 ? (kw <= 26 ? 26 : kw <= 38 ? 38 : 64) : kw <= 8 ? 8 : kw <= 16 ? 16 : 32;
    // (tiles of 32 samples up to 512 features while two workgroups fit a compute unit, of 16 beyond:
    // the instantiated kernels; measured at 2e6 x 100: tiles of 64 samples, which leave room for two
    // workgroups per compute unit instead of four, are no faster)
    // (beyond 128 features tiles of 16 samples, which arrive in LDS directly where there is a row-major
    // copy: four workgroups of four waves per compute unit up to 512 features, two of eight beyond)
    for (int s_log = (nw == 4 && kw_t <= 8) ? 5 : 4; s_log >= (kw_t <= 8 ? 5 : 4); --s_log) {
        const int S = 1 << s_log;
        const size_t lds = fewk_lds(d, S, nw).total;
        const int pieces = (d * (S / 4) + 64 * nw - 1) / (64 * nw);
        // (a larger tile only while two workgroups still fit a compute unit)
        const size_t cap = s_log > 4 ? (size_t)78 * 1024 : (size_t)156 * 1024;
        if (lds <= cap && pieces <= fewk_prefetch(kw_t, s_log, nw)) {
            const int by_lds = (int)((size_t)160 * 1024 / (lds + 512));
            // workgroups per compute unit the kernel's registers allow (waves per SIMD it is built for)
            const bool direct = s_log == 4 && (nw == 4 || kw_t != 38);
            const int by_regs = fewk_waves_per_simd(kw_t, s_log, nw, direct ? 1 : 0) * 4 / nw;
            const int per_cu = by_lds < by_regs ? by_lds : by_regs;
            out->s_log = s_log;
            out->kw = kw_t;
            out->nw = nw;
            out->per_cu = per_cu < 1 ? 1 : per_cu;
            out->lds = lds;
            return true;
        }
    }
    return false;
}

}  // namespace

bool kmx_fewk_supported(int d, int k) {
    FewkShape sh;
    return fewk_shape(d, k, &sh);
}

// room for the partial sums of the largest grid (four workgroups per compute unit)
size_t kmx_fewk_partial_bytes(int d, int k) {
    FewkShape sh;
    if (!fewk_shape(d, k, &sh)) return 0;
    // (a fixed number of compute units: the layout of the workspace is a function of the shape alone;
    // on a larger device the grid stops at what fits)
    const size_t by_workgroup = (size_t)sh.per_cu * 256 * sh.nw * (sh.kw / 4 + 1) * 256 * sizeof(float);
    // (up to 128 features the per-wave kernel may run instead: three workgroups per compute unit, a
    // partial each of up to nine feature blocks)
    const size_t by_wave = d <= 128 ? (size_t)3 * 256 * 9 * 256 * sizeof(float) : 0;
    return by_workgroup > by_wave ? by_workgroup : by_wave;
}

int kmx_fewk_grid(int64_t n, int d, int k, int wgs_per_cu) {
    FewkShape sh;
    if (!fewk_shape(d, k, &sh)) return 1;
    const int64_t tiles = (n + (1 << sh.s_log) - 1) >> sh.s_log;
    int64_t grid = (int64_t)(wgs_per_cu > 0 && wgs_per_cu < sh.per_cu ? wgs_per_cu : sh.per_cu) * kmx_num_cus();
    if (grid > tiles) grid = tiles;
    return grid < 1 ? 1 : (int)grid;
}

// One iteration: the fused step, whose last workgroup also finishes the iteration.  The
// workspace holds the fixed-point exponents and the cleared sums of kmx_lloyd_mfma_prepare.
int32_t kmx_lloyd_iter_fewk(const LloydLayout& L, const void* X_t, const void* X_rowmajor, const void* w,
                            const void* centroids_t, void* new_centroids_t, const uint32_t* labels_prev,
                            uint32_t* labels, void* sizes, uint32_t* empty_clusters, char* ws, int64_t n, int d,
                            int k, hipStream_t stream, hipEvent_t* events) {
    FewkShape sh;
    if (!fewk_shape(d, k, &sh)) return KMX_ERR_UNSUPPORTED;
    LloydTail<float> tail;
    tail.sums_t = (float*)new_centroids_t;
    tail.sizes = (float*)sizes;
    tail.empty_clusters = empty_clusters;
    tail.old_centroids_t = (const float*)centroids_t;
    tail.cpack = nullptr;  // (the packed copy of the centroids is not read by this step's kernels)
    tail.half_norms = reinterpret_cast<float*>(ws + L.off_half);
    tail.status = reinterpret_cast<kmx_lloyd_status*>(ws + L.off_status);
    tail.d = d;
    tail.k = k;
    tail.dpad = L.dpad;
    const int* q_exp = reinterpret_cast<const int*>(ws + L.off_scales) + (d + 1);
    unsigned long long* gsum = reinterpret_cast<unsigned long long*>(ws + L.off_gsum);
    kmx_lloyd_status* status = tail.status;
    const float* half_norms = tail.half_norms;
    float* partial = reinterpret_cast<float*>(ws + L.off_partial);
    int grid = kmx_fewk_grid(n, d, k, L.wgs_per_cu);
    const size_t slots = (size_t)sh.nw * (sh.kw / 4 + 1) * 256;  // partial sums of a workgroup of the instantiated kernel
    if ((size_t)grid * slots * sizeof(float) > L.partial_bytes) grid = (int)(L.partial_bytes / (slots * sizeof(float)));
    if (grid < 1) return KMX_ERR_WORKSPACE;
    const int vec_ok = (n % 4 == 0) && ((((uintptr_t)X_t) & 15) == 0);
    // whole samples from the row-major copy when there is one whose rows are multiples of 16 bytes
    const bool rm = X_rowmajor != nullptr && d % 4 == 0 && ((((uintptr_t)X_rowmajor) & 15) == 0);
    if (events) (void)hipEventRecord(events[0], stream);
    const size_t tail_lds = (size_t)(d + 1) * k * sizeof(float);
#define KMX_FEWK_REDUCE(FBW_, PW_, NW_, N_PARTIALS)                                                        \
    do {                                                                                                  \
        if (tail_lds > 64 * 1024) {                                                                       \
            const hipError_t e =                                                                          \
                hipFuncSetAttribute(reinterpret_cast<const void*>(&fewk_reduce_kernel<FBW_, PW_, NW_>),   \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)tail_lds);           \
            if (e != hipSuccess) return (int32_t)e;                                                       \
        }                                                                                                 \
        hipLaunchKernelGGL((fewk_reduce_kernel<FBW_, PW_, NW_>),                                          \
                           dim3((unsigned)(((PW_ ? 1 : NW_) * FBW_ * 256 + 31) / 32)), dim3(1024), tail_lds, \
                           stream, partial, N_PARTIALS, gsum, q_exp, d, k, tail);                         \
    } while (0)
    if (rm && d <= 128) {
        // every wave on tiles of its own (no barriers): three workgroups per compute unit
        const int nfb = (d + 1 + 15) / 16;
        const int nfb_t = nfb <= 5 ? 5 : nfb <= 7 ? 7 : 9;
        const size_t wave_lds = (size_t)4 * 16 * fewk_wave_ds(fewk_wave_cols(d, nfb_t)) * sizeof(float);
        int64_t wgrid = (int64_t)(L.wgs_per_cu > 0 && L.wgs_per_cu < 3 ? L.wgs_per_cu : 3) * kmx_num_cus();
        const int64_t by_room = (int64_t)(L.partial_bytes / ((size_t)nfb_t * 256 * sizeof(float)));
        const int64_t by_tiles = kmx_cdiv(kmx_cdiv(n, 16), 4);
        if (wgrid > by_room) wgrid = by_room;
        if (wgrid > by_tiles) wgrid = by_tiles;
        if (wgrid < 1) return KMX_ERR_WORKSPACE;
#define KMX_FEWK_WAVE(KS_, NFB_)                                                                           \
    do {                                                                                                  \
        hipLaunchKernelGGL((lloyd_fewk_wave_kernel<KS_, NFB_>), dim3((unsigned)wgrid), dim3(256), wave_lds, \
                           stream, (const float*)X_rowmajor, (const float*)w, (const float*)centroids_t,  \
                           half_norms, labels_prev, labels, partial, status, n, d, k);                    \
        KMX_LAUNCH_CHECK();                                                                               \
        if (events) (void)hipEventRecord(events[1], stream);                                              \
        KMX_FEWK_REDUCE(NFB_, true, 4, (int)wgrid);                                                       \
    } while (0)
        if (nfb_t == 5) KMX_FEWK_WAVE(20, 5);
        else if (nfb_t == 7) KMX_FEWK_WAVE(28, 7);
        else KMX_FEWK_WAVE(32, 9);
#undef KMX_FEWK_WAVE
    } else {
#define KMX_FEWK_LAUNCH_RM(KW_, SL_, RM_, NW_)                                                             \
    do {                                                                                                  \
        constexpr int direct_ = (RM_ && SL_ == 4 && (NW_ == 4 || KW_ != 38)) ? 1 : 0;                     \
        if (sh.lds > 64 * 1024) {                                                                         \
            const hipError_t e = hipFuncSetAttribute(                                                     \
                reinterpret_cast<const void*>(&lloyd_fewk_kernel<KW_, SL_, RM_, NW_, direct_>),           \
                hipFuncAttributeMaxDynamicSharedMemorySize, (int)sh.lds);                                 \
            if (e != hipSuccess) return (int32_t)e;                                                       \
        }                                                                                                 \
        hipLaunchKernelGGL((lloyd_fewk_kernel<KW_, SL_, RM_, NW_, direct_>), dim3((unsigned)grid),        \
                           dim3(64 * NW_),                                                                \
                           sh.lds, stream, (const float*)X_t, (const float*)X_rowmajor, (const float*)w,  \
                           (const float*)centroids_t, half_norms, labels_prev, labels, partial, status,   \
                           n, d, k, vec_ok);                                                              \
    } while (0)
#define KMX_FEWK_LAUNCH(KW_, SL_, FBW_, NW_)                                \
    do {                                                                   \
        if (rm)                                                            \
            KMX_FEWK_LAUNCH_RM(KW_, SL_, true, NW_);                       \
        else                                                               \
            KMX_FEWK_LAUNCH_RM(KW_, SL_, false, NW_);                      \
        KMX_LAUNCH_CHECK();                                                \
        if (events) (void)hipEventRecord(events[1], stream);               \
        KMX_FEWK_REDUCE(FBW_, false, NW_, grid);                           \
    } while (0)
        if (sh.nw == 4 && sh.kw == 8 && sh.s_log == 5) KMX_FEWK_LAUNCH(8, 5, 3, 4);
        else if (sh.nw == 4 && sh.kw == 16 && sh.s_log == 4) KMX_FEWK_LAUNCH(16, 4, 5, 4);
        else if (sh.nw == 4 && sh.kw == 32 && sh.s_log == 4) KMX_FEWK_LAUNCH(32, 4, 9, 4);
        else if (sh.nw == 8 && sh.kw == 26 && sh.s_log == 4) KMX_FEWK_LAUNCH(26, 4, 7, 8);
        else if (sh.nw == 8 && sh.kw == 38 && sh.s_log == 4) KMX_FEWK_LAUNCH(38, 4, 10, 8);
        else if (sh.nw == 8 && sh.kw == 64 && sh.s_log == 4) KMX_FEWK_LAUNCH(64, 4, 17, 8);
        else return KMX_ERR_UNSUPPORTED;
#undef KMX_FEWK_LAUNCH_RM
#undef KMX_FEWK_LAUNCH
    }
#undef KMX_FEWK_REDUCE
    KMX_LAUNCH_CHECK();
    if (events) {
        (void)hipEventRecord(events[2], stream);
        (void)hipEventRecord(events[3], stream);
    }
    return KMX_OK;
}

// Labels only for the shapes of this step (kmx_assign_labels), from the feature-major array.
int32_t kmx_assign_labels_fewk(const void* X_t, const void* centroids_t, const void* half_norms, uint32_t* labels,
                               int64_t n, int d, int k, hipStream_t stream) {
    if (!kmx_fewk_supported(d, k)) return KMX_ERR_UNSUPPORTED;
    // tiles of 64 samples; of 32 while those would not give every compute unit a few tiles
    const int64_t tiles64 = kmx_cdiv(n, 64);
    if (d <= 128 && tiles64 >= (int64_t)16 * kmx_num_cus()) {
        // every wave on tiles of its own (labels are written 128 bits at a time: 16-byte aligned)
        const int vec = (n % 4 == 0) && ((((uintptr_t)X_t) & 15) == 0) && ((((uintptr_t)labels) & 15) == 0);
        int64_t wg = (int64_t)3 * kmx_num_cus();
        if (wg > kmx_cdiv(tiles64, 4)) wg = kmx_cdiv(tiles64, 4);
        hipLaunchKernelGGL((fewk_labels_wave_kernel<32>), dim3((unsigned)wg), dim3(256), 0, stream, (const float*)X_t,
                           (const float*)centroids_t, (const float*)half_norms, labels, n, d, k, vec);
        KMX_LAUNCH_CHECK();
        return KMX_OK;
    }
    const bool small = tiles64 < (int64_t)8 * kmx_num_cus();
    const int ts = small ? 32 : 64;
    const int sv = ts / 16;
    const int vec_ok = (n % sv == 0) && ((((uintptr_t)X_t) & (size_t)(4 * sv - 1)) == 0);
    int64_t grid = (int64_t)2 * kmx_num_cus();
    const int64_t tiles = kmx_cdiv(n, ts);
    if (grid > tiles) grid = tiles;
#define KMX_FEWK_LABELS(KW_, SV_)                                                                                     \
    hipLaunchKernelGGL((fewk_labels_kernel<KW_, SV_>), dim3((unsigned)grid), dim3(512), 0, stream, (const float*)X_t, \
                       (const float*)centroids_t, (const float*)half_norms, labels, n, d, k, vec_ok)
    const int kw = fewk_kw(d, 8);
    if (kw <= 16) {
        if (small) KMX_FEWK_LABELS(16, 2);
        else KMX_FEWK_LABELS(16, 4);
    } else if (kw <= 26) {
        if (small) KMX_FEWK_LABELS(26, 2);
        else KMX_FEWK_LABELS(26, 4);
    } else if (kw <= 38) {
        if (small) KMX_FEWK_LABELS(38, 2);
        else KMX_FEWK_LABELS(38, 4);
    } else {
        if (small) KMX_FEWK_LABELS(64, 2);
        else KMX_FEWK_LABELS(64, 4);
    }
#undef KMX_FEWK_LABELS
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
