// Label step of the wide fp32 Lloyd path (samples in registers, centroids streamed through
// LDS; see lloyd_mfma_wide.hip) with the scores SCREENED on the fp16 matrix cores and certified
// per sample, as in lloyd_mfma_screen.hip:
//
//   * X and the centroids are scaled by the power of two that brings max|x| into [2^14, 2^15)
//     and split into two fp16 parts each; score ~ hi*hi + lo*hi + hi*lo accumulated in fp32
//     from -0.5||c||^2: 3 v_mfma_f32_32x32x16_f16 (96 cycles) per 32 centroids x 32 samples x
//     16 features instead of 8 v_mfma_f32_32x32x2_f32 (512 cycles).
//   * Error of one score: the split leaves out at most 3.01 * 2^-22 * sum_f |x_f c_f| (plus
//     2^-14 per element in absolute terms, which covers flushed fp16 subnormals); the fp32
//     accumulation of the 48 exact products per 16 features adds at most 51 roundings of one
//     ulp of a partial sum per K step.  With R = 51 * ceil(d / 16) roundings,
//       E(x) = (7.2e-7 + R 2^-23) ||x|| C + R 2^-23 H + 6.2e-5 sqrt(d) (||x|| + C),
//     C = max ||c||, H = max 0.5||c||^2 (scaled units).  best - second > 2 E(x) certifies the
//     label; any other sample goes on a list, and the all-fp32 label kernel of
//     lloyd_mfma_wide.hip runs on the listed samples afterwards (k * d multiply-adds per sample
//     are only affordable on the matrix cores, with the centroids shared by a whole tile).
//   * The fp16 parts of the centroids are prepared once per iteration by wide_split_kernel in
//     the order the label kernel consumes them (per chunk of 128 centroids x 32 features: block,
//     K step, part, lane -> 8 halves), so a chunk is a plain 16 KB copy into LDS and every A
//     operand one 128-bit LDS read.
//
// Only the counting mode of the wide path is covered (labels, changed count, per-cluster counts
// and ranks; the sums are taken by the bucketed accumulation from the row-major copy of X).
#include "lloyd_layout.h"

#include <type_traits>

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef double v8d __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

constexpr int KC = 32;   // features per chunk (two K steps of 16)
constexpr int CG = 128;  // centroids per chunk (four MFMA blocks)
constexpr int CHUNK_VEC = 4 * 2 * 2 * 64;  // 16-byte entries per chunk: block, K step, part, lane
constexpr int G = 8;     // accumulator registers per arg-max group

constexpr float WS_ERR_SPLIT = 7.2e-7f;   // 3.01 * 2^-22, rounded up
constexpr float WS_ERR_ROUND = 1.2e-7f;   // 2^-23, rounded up
constexpr float WS_ERR_ABS = 6.2e-5f;     // 2^-14, rounded up

// LDS reads the compiler must not see as LDS reads: after a direct global-to-LDS load it puts a
// wait for ALL outstanding loads in front of every LDS read it knows of (it cannot tell which
// buffer the load fills), which would serialise the chunk pipeline.  The values are only valid
// after lds_wait(), which takes them as operands so that no consumer is scheduled before it.
typedef float v4f __attribute__((ext_vector_type(4)));
template <int OFFSET>
__device__ __forceinline__ v4f lds_read16(unsigned int addr) {
    v4f v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
__device__ __forceinline__ void lds_wait(v4f& a, v4f& b, v4f& c, v4f& d) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
// the same with the four most recent reads still in flight (a, b, c, d were issued before them)
__device__ __forceinline__ void lds_wait_but4(v4f& a, v4f& b, v4f& c, v4f& d) {
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// header words in the workspace
constexpr int HDR_HMAX = 0;       // bits of max 0.5||c * scale||^2
constexpr int HDR_SCALE = 1;      // bits of the scale
constexpr int HDR_UNCERTAIN = 2;  // samples evaluated in fp32 by the last label step
constexpr int HDR_TILE = 3;       // tiles handed out beyond the first one of every workgroup

// fp16 parts of the scaled centroids in consumption order, scaled -0.5||c||^2, and the header.
// One thread per (chunk, block, K step, lane); launched with enough blocks of 256 threads.
__global__ __launch_bounds__(256) void wide_split_kernel(const float* __restrict__ centroids_t,
                                                         const unsigned int* __restrict__ absmax,
                                                         uint4* __restrict__ split,
                                                         float* __restrict__ hneg,
                                                         unsigned int* __restrict__ header, int d, int k,
                                                         int nkc, int n_cg) {
    __shared__ float xs_s;
    if (threadIdx.x < 64) {
        float m = 0.0f;
        for (int f = threadIdx.x; f < d; f += 64) m = fmaxf(m, __uint_as_float(absmax[f]));
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        if (threadIdx.x == 0) xs_s = (m > 0.0f && m < kmx_inf<float>()) ? ldexpf(1.0f, 14 - ilogbf(m)) : 1.0f;
    }
    __syncthreads();
    const float xs = xs_s;
    const int total = n_cg * nkc * 4 * 2 * 64;
    for (int idx = blockIdx.x * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
        const int l = idx & 63;
        const int s2 = (idx >> 6) & 1;
        const int b = (idx >> 7) & 3;
        const int chunk = idx >> 9;  // cg * nkc + kc
        const int kc = chunk % nkc, cg = chunk / nkc;
        const int c = cg * CG + 32 * b + (l & 31);
        v8h hi, lo;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int f = kc * KC + 16 * s2 + 2 * i + (l >> 5);
            const float v = (c < k && f < d) ? centroids_t[(size_t)f * k + c] * xs : 0.0f;
            const _Float16 hb = (_Float16)v;
            hi[i] = hb;
            lo[i] = (_Float16)(v - (float)hb);
        }
        uint4* dst = split + (size_t)chunk * CHUNK_VEC + ((b * 2 + s2) * 2) * 64 + l;
        dst[0] = __builtin_bit_cast(uint4, hi);
        dst[64] = __builtin_bit_cast(uint4, lo);
    }
    // -0.5||c||^2 of the scaled centroids: 64 centroids per workgroup and pass, the features in
    // four interleaved slices (one per wave) whose partial sums are added in a fixed order
    __shared__ float part_s[4][64];
    const int cl = threadIdx.x & 63, fs = threadIdx.x >> 6;
    for (int c0 = blockIdx.x * 64; c0 < n_cg * CG; c0 += gridDim.x * 64) {
        const int c = c0 + cl;
        float sq = 0.0f;
        if (c < k) {
            for (int f = fs; f < d; f += 4) {
                const float cv = centroids_t[(size_t)f * k + c] * xs;
                sq += cv * cv;
            }
        }
        part_s[fs][cl] = sq;
        __syncthreads();
        if (fs == 0) {
            float v = -kmx_inf<float>();
            if (c < k) {
                const float tot = (part_s[0][cl] + part_s[1][cl]) + (part_s[2][cl] + part_s[3][cl]);
                v = -(tot / 2.0f);
                atomicMax(header + HDR_HMAX, __float_as_uint(tot / 2.0f));
            }
            hneg[c] = v;
        }
        __syncthreads();
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) header[HDR_SCALE] = __float_as_uint(xs);
}

__global__ void wide_header_reset_kernel(unsigned int* header) {
    if (threadIdx.x == 0) {
        header[HDR_HMAX] = 0u;
        header[HDR_UNCERTAIN] = 0u;
        header[HDR_TILE] = 0u;
    }
}

template <int NKC>
__global__ __launch_bounds__(256, 2) void lloyd_wide_screen_kernel(
    const float* __restrict__ X_t, const uint4* __restrict__ split, const float* __restrict__ hneg,
    unsigned int* __restrict__ header, int* __restrict__ list,
    const uint32_t* __restrict__ labels_prev, uint32_t* __restrict__ labels,
    kmx_lloyd_status* __restrict__ status, int* __restrict__ counts, int* __restrict__ ranks,
    int64_t n, int d, int k) {
    // labels only: no status, previous labels, counts or ranks
    const bool update = status != nullptr;
    if (update && status->state != KMX_RUNNING) return;

    constexpr int NS = 2 * NKC;  // K steps of 16 features
    __shared__ __align__(16) uint4 ctile[3][CHUNK_VEC];
    extern __shared__ __align__(16) float hneg_s[];    // [n_cg * CG]
    __shared__ unsigned int changed_block;

    const int n_cg = (k + CG - 1) / CG;
    for (int c = threadIdx.x; c < n_cg * CG; c += 256) hneg_s[c] = hneg[c];
    if (threadIdx.x == 0) changed_block = 0;

    // (the wave index as a scalar: what is derived from it, such as the LDS base of the chunk
    // copies, then needs no vector instructions)
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int h = lane >> 5, j = lane & 31;
    const int64_t n_tiles = (n + 127) >> 7;
    unsigned int changed = 0;

    const float xs = __uint_as_float(header[HDR_SCALE]);
    const float hmax = __uint_as_float(header[HDR_HMAX]);
    const float cmax = sqrtf(2.0f * hmax);
    const float round_term = WS_ERR_ROUND * 51.0f * (float)((d + 15) / 16);
    const float abs_term = WS_ERR_ABS * sqrtf((float)d);
    const float thr_x = 2.01f * ((WS_ERR_SPLIT + round_term) * cmax + abs_term);
    const float thr_0 = 2.01f * (round_term * hmax + abs_term * cmax);
    float pos_inf = kmx_inf<float>();
    asm volatile("" : "+s"(pos_inf));  // see lloyd_mfma_screen.hip: keeps the median below a median
    const float neg_inf = -kmx_inf<float>();

    // Chunk copy, straight from global memory into LDS (no registers held while the data are in
    // flight, so a chunk can be requested two steps ahead): thread t moves entries t, t + 256,
    // t + 512, t + 768 of the 1024; the LDS address of such a load is a per-wave base plus
    // 16 bytes per lane.
    const int n_chunks = n_cg * NKC;
    // LDS byte addresses of the lane's 16 bytes in chunk buffer 0 and of -0.5||c||^2
    const unsigned int tile_addr = (unsigned int)(uintptr_t)(&ctile[0][0]) + (unsigned int)lane * 16u;
    const unsigned int hneg_addr = (unsigned int)(uintptr_t)(&hneg_s[0]);
    auto chunk_issue = [&](int chunk, int buf) {
        const uint4* __restrict__ src = split + (size_t)chunk * CHUNK_VEC + 64 * wave + lane;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            __builtin_amdgcn_global_load_lds(
                src + 256 * q, (__attribute__((address_space(3))) void*)(&ctile[buf][256 * q + 64 * wave]), 16, 0, 0);
    };

    // Tiles beyond the first are drawn from a counter in memory (a tile takes tens of
    // microseconds, the draw is requested during the X loads and published by the barrier the
    // tile needs anyway): with fixed shares the workgroups with one tile more than the others
    // set the time.
    __shared__ unsigned int next_tile_s;
    for (int64_t tile = blockIdx.x; tile < n_tiles;) {
        unsigned int drawn = 0;
        if (threadIdx.x == 0) drawn = atomicAdd(header + HDR_TILE, 1u);
        const int64_t i = tile * 128 + wave * 32 + j;
        const bool valid = i < n;

        // features 16 S + 2 q + h of sample j, scaled and split; ||x||^2 on the way
        v8h xh[NS], xl[NS];
        float ss = 0.0f;
        {
            // Loaded in batches of eight K steps, 64 values in flight per lane, then converted.
            // The loads are inline assembly: at this register pressure the compiler would
            // otherwise funnel every value through one register and wait for each load in turn,
            // paying the memory latency 128 times per tile.  The values are valid after the wait
            // statement, which takes them as operands.
            // Every load is a scalar row address plus a 32-bit byte offset of the lane (n < 2^29):
            // no vector instruction goes into addresses.  Which rows exist is the same for the
            // whole wave and decided by scalar branches (the assembly in their bodies keeps the
            // compiler from turning them into per-lane selects): a pair below d reads rows f0
            // and f0 + 1; of a last pair that is half there (odd d) both half-waves read row
            // d - 1 and the upper one drops the value; a pair past d reads row 0 and is scaled
            // by zero.  A lane past the end works on sample 0 and its results are not used.
            const uint32_t off_0 = (uint32_t)(valid ? i : 0) * 4u;
            const uint32_t off_h = off_0 + (uint32_t)h * (uint32_t)n * 4u;
            const size_t pair_stride = (size_t)n * 8u;  // two rows
            auto load_batch = [&](auto s0_tag, auto batch_tag) {
                constexpr int S0 = decltype(s0_tag)::value, BATCH = decltype(batch_tag)::value;
                static_assert(BATCH % 2 == 0, "the wait statements take 16 values each");
                float raw[BATCH * 8];
                // (d and the base are hidden from loop-invariant hoisting: one lane mask and one
                // 64-bit pointer per row kept across the tile loop would all be spilled)
                int d_now = d;
                size_t hidden_zero = 0;
                asm volatile("" : "+s"(d_now), "+s"(hidden_zero));
                const char* row = reinterpret_cast<const char*>(X_t) + hidden_zero + (size_t)(8 * S0) * pair_stride;
#pragma unroll
                for (int u = 0; u < BATCH * 8; ++u) {
                    const int f0 = 16 * S0 + 2 * u;  // the pair's even feature
                    if (f0 + 1 < d_now) {
                        asm volatile("global_load_dword %0, %1, %2" : "=v"(raw[u]) : "v"(off_h), "s"(row));
                    } else {
                        const char* one_row = f0 < d_now ? row : reinterpret_cast<const char*>(X_t);
                        asm volatile("global_load_dword %0, %1, %2" : "=v"(raw[u]) : "v"(off_0), "s"(one_row));
                    }
                    row += pair_stride;
                }
                // one wait for the whole batch; the statements take 16 values each (operand limit)
#pragma unroll
                for (int g = 0; g < BATCH * 8; g += 16)
                    asm volatile("s_waitcnt vmcnt(0)"
                                 : "+v"(raw[g + 0]), "+v"(raw[g + 1]), "+v"(raw[g + 2]), "+v"(raw[g + 3]),
                                   "+v"(raw[g + 4]), "+v"(raw[g + 5]), "+v"(raw[g + 6]), "+v"(raw[g + 7]),
                                   "+v"(raw[g + 8]), "+v"(raw[g + 9]), "+v"(raw[g + 10]), "+v"(raw[g + 11]),
                                   "+v"(raw[g + 12]), "+v"(raw[g + 13]), "+v"(raw[g + 14]), "+v"(raw[g + 15]));
                float scaled[BATCH * 8];
                int d_then = d;  // compared afresh again: nothing kept from the loads above
                asm volatile("" : "+s"(d_then));
#pragma unroll
                for (int u = 0; u < BATCH * 8; ++u) {
                    const int f0 = 16 * S0 + 2 * u;
                    scaled[u] = raw[u] * xs;
                    if (f0 + 1 >= d_then) {  // the last pair of an odd d, or padding
                        asm volatile("" : "+v"(scaled[u]));
                        if (f0 >= d_then || h) scaled[u] = 0.0f;
                    }
                }
#pragma unroll
                for (int u = 0; u < BATCH * 8; u += 2) {
                    const int S = S0 + u / 8, q = u % 8;
                    const v2f p = {scaled[u], scaled[u + 1]};
                    const v2h hh = __builtin_convertvector(p, v2h);
                    const v2f r = p - __builtin_convertvector(hh, v2f);
                    const v2h ll = __builtin_convertvector(r, v2h);
                    xh[S][q] = hh[0];
                    xh[S][q + 1] = hh[1];
                    xl[S][q] = ll[0];
                    xl[S][q + 1] = ll[1];
                    ss = fmaf(p[0], p[0], ss);
                    ss = fmaf(p[1], p[1], ss);
                }
            };
            constexpr int FULL8 = NS / 8, REST = NS % 8;  // NS is even
            if constexpr (FULL8 >= 1) load_batch(std::integral_constant<int, 0>{}, std::integral_constant<int, 8>{});
            if constexpr (FULL8 >= 2) load_batch(std::integral_constant<int, 8>{}, std::integral_constant<int, 8>{});
            static_assert(FULL8 <= 2, "d <= 256");
            if constexpr (REST > 0)
                load_batch(std::integral_constant<int, 8 * FULL8>{}, std::integral_constant<int, REST>{});
        }
        const float nrm = ss + __shfl_xor(ss, 32, 64);

        float best = neg_inf, second = neg_inf;
        unsigned int code = 0;
        double s0, s1, s2, s3;  // the winning group's registers, as pairs
        asm volatile("" : "=v"(s0), "=v"(s1), "=v"(s2), "=v"(s3));

        if (threadIdx.x == 0) next_tile_s = gridDim.x + drawn;
        __syncthreads();  // every wave is done with the LDS buffers (previous tile); hneg_s is set
        const int64_t tile_after = (int64_t)next_tile_s;  // rewritten only after the barriers of this tile
        chunk_issue(0, 0);
        if (n_chunks > 1) chunk_issue(1, 1);

        for (int cg = 0; cg < n_cg; ++cg) {
            // accumulator register r of half-wave h is centroid 8 (r / 4) + 4 h + r % 4 of the block
            v16f acc[4];
            {
                const unsigned int hb = hneg_addr + (unsigned int)(cg * CG + 4 * h) * 4u;
#define KMX_HNEG_BLOCK(B)                                                                  \
    {                                                                                      \
        v4f q0 = lds_read16<(32 * B) * 4>(hb), q1 = lds_read16<(32 * B + 8) * 4>(hb);        \
        v4f q2 = lds_read16<(32 * B + 16) * 4>(hb), q3 = lds_read16<(32 * B + 24) * 4>(hb);  \
        lds_wait(q0, q1, q2, q3);                                                          \
        _Pragma("unroll") for (int e = 0; e < 4; ++e) {                                    \
            acc[B][e] = q0[e];                                                             \
            acc[B][4 + e] = q1[e];                                                         \
            acc[B][8 + e] = q2[e];                                                         \
            acc[B][12 + e] = q3[e];                                                        \
        }                                                                                  \
    }
                KMX_HNEG_BLOCK(0)
                KMX_HNEG_BLOCK(1)
                KMX_HNEG_BLOCK(2)
                KMX_HNEG_BLOCK(3)
#undef KMX_HNEG_BLOCK
            }
#pragma unroll
            for (int kc = 0; kc < NKC; ++kc) {
                const int step = cg * NKC + kc;
                // this wave's loads of chunk `step` are complete when at most the four of chunk
                // step + 1 are outstanding; the barrier then makes every wave's part visible and
                // tells that all waves are done with chunk step - 1, whose buffer chunk step + 2
                // may overwrite
                if (step + 1 < n_chunks)
                    asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (step + 2 < n_chunks) chunk_issue(step + 2, (step + 2) % 3);
                const unsigned int fa = tile_addr + (unsigned int)(step % 3) * (CHUNK_VEC * 16u);
                // Entry ((b * 2 + s2) * 2 + part) * 64 + lane of the chunk, 16 bytes each.  The
                // four blocks are independent chains: their MFMAs are interleaved so that none
                // waits for the result of the one before it.  The LDS reads run one group of
                // MFMAs ahead (LDS reads of a wave complete in order): the hi parts of a K
                // step are used while its lo parts arrive, the lo parts while the next hi parts
                // arrive; a register is reloaded once the MFMAs reading it have been issued.
                v4f rh[4], rl[4];
                auto read_hi = [&](auto s_tag) {
                    constexpr int S2 = decltype(s_tag)::value;
                    rh[0] = lds_read16<(0 + 2 * S2) * 1024>(fa);
                    rh[1] = lds_read16<(4 + 2 * S2) * 1024>(fa);
                    rh[2] = lds_read16<(8 + 2 * S2) * 1024>(fa);
                    rh[3] = lds_read16<(12 + 2 * S2) * 1024>(fa);
                };
                auto read_lo = [&](auto s_tag) {
                    constexpr int S2 = decltype(s_tag)::value;
                    rl[0] = lds_read16<(1 + 2 * S2) * 1024>(fa);
                    rl[1] = lds_read16<(5 + 2 * S2) * 1024>(fa);
                    rl[2] = lds_read16<(9 + 2 * S2) * 1024>(fa);
                    rl[3] = lds_read16<(13 + 2 * S2) * 1024>(fa);
                };
                auto mfma_hi = [&](const int S) {  // hi * hi, hi * lo
                    v8h ah[4];
#pragma unroll
                    for (int b = 0; b < 4; ++b) ah[b] = __builtin_bit_cast(v8h, rh[b]);
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[b], xh[S], acc[b], 0, 0, 0);
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[b], xl[S], acc[b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                };
                auto mfma_lo = [&](const int S) {  // lo * hi
                    v8h al[4];
#pragma unroll
                    for (int b = 0; b < 4; ++b) al[b] = __builtin_bit_cast(v8h, rl[b]);
#pragma unroll
                    for (int b = 0; b < 4; ++b)
                        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al[b], xh[S], acc[b], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                };
                using Step0 = std::integral_constant<int, 0>;
                using Step1 = std::integral_constant<int, 1>;
                read_hi(Step0{});
                read_lo(Step0{});
                lds_wait_but4(rh[0], rh[1], rh[2], rh[3]);
                mfma_hi(2 * kc);
                lds_wait(rl[0], rl[1], rl[2], rl[3]);
                read_hi(Step1{});
                mfma_lo(2 * kc);
                read_lo(Step1{});
                lds_wait_but4(rh[0], rh[1], rh[2], rh[3]);
                mfma_hi(2 * kc + 1);
                lds_wait(rl[0], rl[1], rl[2], rl[3]);
                mfma_lo(2 * kc + 1);
            }

            // arg-max by groups of 8 registers with the second largest of the group maxima
#pragma unroll
            for (int b = 0; b < 4; ++b)
#pragma unroll
                for (int g = 0; g < 2; ++g) {
                    const unsigned int cd = (unsigned int)(cg * 8 + b * 2 + g);  // wave-uniform
                    float m = __builtin_amdgcn_fmed3f(acc[b][g * G], acc[b][g * G + 1], pos_inf);
#pragma unroll
                    for (int r = 2; r + 1 < G; r += 2)
                        asm("v_max3_f32 %0, %1, %2, %3"
                            : "=v"(m)
                            : "v"(m), "v"(acc[b][g * G + r]), "v"(acc[b][g * G + r + 1]));
                    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(second) : "v"(best), "v"(second), "v"(m));
                    if (m > best) {  // strict: the earlier group keeps a tie
                        best = m;
                        code = cd;
                        const v8d ad = __builtin_bit_cast(v8d, acc[b]);
                        asm volatile("v_mov_b64 %0, %1" : "+v"(s0) : "v"(ad[g * 4]));
                        asm volatile("v_mov_b64 %0, %1" : "+v"(s1) : "v"(ad[g * 4 + 1]));
                        asm volatile("v_mov_b64 %0, %1" : "+v"(s2) : "v"(ad[g * 4 + 2]));
                        asm volatile("v_mov_b64 %0, %1" : "+v"(s3) : "v"(ad[g * 4 + 3]));
                    }
                }
        }

        // position inside the winning group, second largest inside it, both half-waves
        float sv[G];
        {
            const float2 p0 = __builtin_bit_cast(float2, s0), p1 = __builtin_bit_cast(float2, s1);
            const float2 p2 = __builtin_bit_cast(float2, s2), p3 = __builtin_bit_cast(float2, s3);
            sv[0] = p0.x; sv[1] = p0.y; sv[2] = p1.x; sv[3] = p1.y;
            sv[4] = p2.x; sv[5] = p2.y; sv[6] = p3.x; sv[7] = p3.y;
        }
        unsigned int pos = G - 1, n_eq = 0;
        float sec = second;
#pragma unroll
        for (int r = G - 1; r >= 0; --r) {
            const bool eq = sv[r] == best;
            pos = eq ? (unsigned int)r : pos;
            n_eq += eq ? 1u : 0u;
            const float rest = eq ? neg_inf : sv[r];
            sec = rest > sec ? rest : sec;
        }
        sec = n_eq > 1u ? best : sec;
        // code = 8 cg + 2 b + g; register = 8 g + pos
        const unsigned int reg = (code & 1u) * G + pos;
        int c = (int)(CG * (code >> 3) + 32 * ((code >> 1) & 3u) + 8 * (reg >> 2) + 4 * h + (reg & 3u));
        float bb = best;
        {
            const float ov = __shfl_xor(best, 32, 64);
            const float o2 = __shfl_xor(sec, 32, 64);
            const int oc = __shfl_xor(c, 32, 64);
            float t2 = sec > o2 ? sec : o2;
            const float lo_best = ov < best ? ov : best;
            sec = lo_best > t2 ? lo_best : t2;
            if (ov > bb || (ov == bb && oc < c)) {
                c = oc;
                bb = ov;
            }
        }
        // written so that a NaN anywhere makes the sample uncertain
        const float thr = fmaf(thr_x, __builtin_amdgcn_sqrtf(nrm), thr_0);
        const bool unsure = !(bb - sec > thr) && valid;

        // samples the screen cannot certify go on the list for the all-fp32 kernel (one atomic
        // per wave and tile that has any)
        const unsigned long long um = __ballot(h == 0 && unsure);
        if (um) {
            unsigned int base = 0;
            if (lane == 0) base = atomicAdd(header + HDR_UNCERTAIN, (unsigned int)__popcll(um));
            base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
            if (h == 0 && unsure) list[base + __popcll(um & ((1ull << lane) - 1ull))] = (int)i;
        }
        const uint32_t lab = (uint32_t)c;

        if (valid && h == 0 && !unsure) {
            labels[i] = lab;
            if (update) {
                changed += (labels_prev[i] != lab) ? 1u : 0u;
                // the returned count is the sample's rank inside its cluster (for the scatter)
                ranks[i] = atomicAdd(counts + lab, 1);
            }
        }
        tile = tile_after;
    }

    if (changed) atomicAdd(&changed_block, changed);
    __syncthreads();
    if (update && threadIdx.x == 0 && changed_block) atomicAdd(&status->n_changed, changed_block);
}

// absmax[f] = bits of 4 max|c| for every feature: the stand-in for max|x| where only the
// centroids are at hand (labels only); one workgroup.
__global__ __launch_bounds__(1024) void wide_scale_from_centroids_kernel(const float* __restrict__ centroids_t,
                                                                        unsigned int* __restrict__ absmax,
                                                                        int d, int k) {
    __shared__ unsigned int m_bits;
    if (threadIdx.x == 0) m_bits = 0u;
    __syncthreads();
    float m = 0.0f;
    for (int idx = threadIdx.x; idx < d * k; idx += 1024) m = fmaxf(m, fabsf(centroids_t[idx]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if ((threadIdx.x & 63) == 0) atomicMax(&m_bits, __float_as_uint(4.0f * m));  // non-negative: ordered like the bits
    __syncthreads();
    for (int f = threadIdx.x; f < d; f += 1024) absmax[f] = m_bits;
}

}  // namespace

int32_t kmx_wide_screen_scale_from_centroids(const void* centroids_t, unsigned int* absmax, int d, int k,
                                             hipStream_t stream) {
    hipLaunchKernelGGL(wide_scale_from_centroids_kernel, dim3(1), dim3(1024), 0, stream,
                       (const float*)centroids_t, absmax, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

size_t kmx_wide_screen_bytes(int64_t n, int d, int k) {
    const size_t n_cg = (size_t)(k + CG - 1) / CG, nkc = (size_t)(d + KC - 1) / KC;
    return 256 + n_cg * CG * sizeof(float) + n_cg * nkc * CHUNK_VEC * sizeof(uint4) + (size_t)n * sizeof(int);
}

// KMX_FLAG_LABELS_F32 switches the screen off (all-fp32 scores, lloyd_mfma_wide.hip).
bool kmx_wide_screen_enabled(int64_t n, int d, int k, uint32_t flags) {
    // (the label kernel addresses a lane's samples with 32-bit byte offsets into two rows)
    if (!kmx_mfma_wide_supported(d, k) || n >= ((int64_t)1 << 29)) return false;
    return (flags & KMX_FLAG_LABELS_MASK) != KMX_FLAG_LABELS_F32;
}

const uint32_t* kmx_wide_screen_counter(const char* area) {
    return reinterpret_cast<const uint32_t*>(area) + HDR_UNCERTAIN;
}

const int* kmx_wide_screen_list(const char* area, int d, int k) {
    const size_t n_cg = (size_t)(k + CG - 1) / CG, nkc = (size_t)(d + KC - 1) / KC;
    return reinterpret_cast<const int*>(area + 256 + n_cg * CG * sizeof(float) +
                                        n_cg * nkc * CHUNK_VEC * sizeof(uint4));
}

// Labels, changed count, per-cluster counts and ranks of the certified samples; the others are
// listed (count in the header word kmx_wide_screen_counter points at, indices at
// kmx_wide_screen_list) for the all-fp32 kernel.  `area`: kmx_wide_screen_bytes of workspace;
// `absmax`: bits of max|X_t row| per feature.
int32_t kmx_lloyd_wide_screen_count(const void* X_t, const void* centroids_t,
                                    const unsigned int* absmax, char* area,
                                    const uint32_t* labels_prev, uint32_t* labels,
                                    kmx_lloyd_status* status, int* counts, int* ranks, int64_t n,
                                    int d, int k, hipStream_t stream) {
    const int n_cg = (k + CG - 1) / CG, nkc = (d + KC - 1) / KC;
    unsigned int* header = reinterpret_cast<unsigned int*>(area);
    float* hneg = reinterpret_cast<float*>(area + 256);
    uint4* split = reinterpret_cast<uint4*>(area + 256 + (size_t)n_cg * CG * sizeof(float));
    int* list = const_cast<int*>(kmx_wide_screen_list(area, d, k));
    hipLaunchKernelGGL(wide_header_reset_kernel, dim3(1), dim3(64), 0, stream, header);
    const int total = n_cg * nkc * 4 * 2 * 64;
    hipLaunchKernelGGL(wide_split_kernel, dim3((unsigned)kmx_cdiv(total, 256)), dim3(256), 0, stream,
                       (const float*)centroids_t, absmax, split, hneg, header, d, k, nkc, n_cg);
    const size_t lds = (size_t)n_cg * CG * sizeof(float);
    int64_t grid = kmx_cdiv(n, 128);
    const int64_t cap = 2 * (int64_t)kmx_num_cus();
    if (grid > cap) grid = cap;
    if (grid < 1) grid = 1;
#define KMX_WS_CASE(NKC)                                                                              \
    hipLaunchKernelGGL((lloyd_wide_screen_kernel<NKC>), dim3((unsigned)grid), dim3(256), lds, stream, \
                       (const float*)X_t, split, hneg, header, list, labels_prev, labels, status,     \
                       counts, ranks, n, d, k)
    switch (nkc) {
        case 1: KMX_WS_CASE(1); break;
        case 2: KMX_WS_CASE(2); break;
        case 3: KMX_WS_CASE(3); break;
        case 4: KMX_WS_CASE(4); break;
        case 5: KMX_WS_CASE(5); break;
        case 6: KMX_WS_CASE(6); break;
        case 7: KMX_WS_CASE(7); break;
        case 8: KMX_WS_CASE(8); break;
        default: return KMX_ERR_UNSUPPORTED;
    }
#undef KMX_WS_CASE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
