// Radix-select top-k of the rows of a float matrix on gfx950 (a 1-D array is one row; KMeans
// uses it to relocate empty clusters onto the samples farthest from their centroid).
//
// Floats are mapped to unsigned keys whose integer order is the float order (-0.0 counts as
// +0.0).  The key of the k-th largest value of a row is fixed digit by digit, most significant
// first; digits are 11 or 10 bits wide (3 digits for fp32, 6 for fp64).  All rows advance
// together: the row is the second grid dimension of every kernel.
//
//   pass 0   reads the row once (128-bit loads), histogram of the first digit in LDS, flushed
//            to the row's global histogram with 64-bit atomics.
//   pass 1   reads the row a second time: keys whose first digit is above the selected one are
//            winners and go straight to the result slots; keys that share it are the
//            candidates: each workgroup appends them to its own segment of a side buffer
//            (an LDS counter, no global atomics) and histograms their second digit.
//   pass 2.. walk the candidates only (typically a few thousand keys); when a segment of the
//            side buffer overflowed (the buffer holds a quarter of the row), they walk the
//            row itself instead.
//   gather   candidates above the threshold key are winners; of the keys equal to it, the
//            lowest indices are taken.
//   order    the k winners are ranked by descending value, then ascending index, so the result
//            is deterministic.
//
// The workgroup that finishes a pass last (a ticket counter per row) walks the histogram from
// the top and fixes the digit, so a pass is one launch and nothing returns to the host.  What
// workgroups exchange inside a launch (histogram, ticket, overflow flag, lowest tie) moves
// through device-scope atomics only, which are performed at the memory side: waiting for them
// to complete orders them, and no cache write-back or invalidation is needed (a full fence
// costs about 60 us per launch here, the L2 of every chiplet being flushed by every workgroup).
#include "kmx_common.h"

namespace {

constexpr int TOPK_WG = 1024;  // few, large workgroups: what they exchange goes through same-address atomics,
                               // which the memory side performs one after the other (10-20 ns each)
constexpr int TOPK_MAX_BUCKETS = 2048;
constexpr unsigned int TOPK_TIE_LIST = 1024;  // indices of keys equal to the threshold kept aside
constexpr int TOPK_WIDE = 11;  // bits of the first digits; the last ones may take 10

struct TopkState {
    unsigned long long prefix;      // digits fixed so far (threshold key after the last pass)
    long long k_rem;                // how many keys equal to the threshold belong to the top k
    unsigned long long n_out;       // winners written so far
    unsigned long long tie_min;     // lowest index holding the threshold key
    unsigned int ticket;            // workgroups that finished the running pass
    unsigned int overflow;          // set by a workgroup whose segment of the side buffer was too small
    unsigned int cand_ok;           // 1: the side buffer holds every candidate
    unsigned int n_ties;            // indices appended to the tie list (may exceed its capacity)
    unsigned int pad[4];
};

constexpr int TOPK_MAX_SEGMENTS = 256;  // workgroups per row of the passes that read the row

struct TopkLayout {
    size_t off_state, off_hist, off_counts, off_keys, off_idx, off_cand_keys, off_cand_idx, off_small, row_bytes;
    int64_t n_seg, seg_cap;  // segments of the side buffer (one per workgroup of pass 1) and their capacity
};

size_t topk_small_bytes(int64_t n, int32_t k);  // (the one-read path for small k, further down)

TopkLayout topk_layout(int64_t rows, int64_t n, int32_t k, int32_t dtype) {
    TopkLayout L;
    const int64_t vec = dtype == KMX_F64 ? 2 : 4;
    // >= 4 loads of 128 bits per lane, and about TOPK_MAX_SEGMENTS workgroups over all rows
    L.n_seg = kmx_cdiv(kmx_cdiv(n + vec, vec), TOPK_WG * 4);
    const int64_t share = kmx_cdiv(TOPK_MAX_SEGMENTS, rows);
    if (L.n_seg > share) L.n_seg = share;
    if (L.n_seg < 1) L.n_seg = 1;
    L.seg_cap = kmx_cdiv(kmx_cdiv(n, 4), L.n_seg);
    if (L.seg_cap < 64) L.seg_cap = 64;
    const size_t cap = (size_t)(L.n_seg * L.seg_cap);
    L.off_state = 0;
    L.off_hist = 256;
    L.off_counts = L.off_hist + TOPK_MAX_BUCKETS * sizeof(unsigned long long);
    L.off_keys = L.off_counts + kmx_align256((size_t)L.n_seg * sizeof(unsigned int));
    L.off_idx = L.off_keys + kmx_align256((size_t)k * sizeof(unsigned long long));
    L.off_cand_keys = L.off_idx + kmx_align256((size_t)k * sizeof(long long));
    L.off_cand_idx = L.off_cand_keys + kmx_align256(cap * kmx_dtype_size(dtype));
    L.off_small = L.off_cand_idx + kmx_align256(cap * sizeof(long long));
    L.row_bytes = L.off_small + topk_small_bytes(n, k);
    return L;
}

// Per-row pointers into the workspace.
struct TopkRow {
    TopkState* st;
    unsigned long long* hist;
    unsigned int* counts;
    unsigned long long* keys;
    long long* idx;
    void* cand_keys;
    long long* cand_idx;
};

struct TopkArgs {
    char* ws;
    size_t row_bytes, off_hist, off_counts, off_keys, off_idx, off_cand_keys, off_cand_idx;
    int64_t n;
    int32_t k, n_seg, seg_cap;
};

__device__ __forceinline__ TopkRow topk_row(const TopkArgs& a, int64_t row) {
    char* base = a.ws + (size_t)row * a.row_bytes;
    TopkRow r;
    r.st = (TopkState*)base;
    r.hist = (unsigned long long*)(base + a.off_hist);
    r.counts = (unsigned int*)(base + a.off_counts);
    r.keys = (unsigned long long*)(base + a.off_keys);
    r.idx = (long long*)(base + a.off_idx);
    r.cand_keys = base + a.off_cand_keys;
    r.cand_idx = (long long*)(base + a.off_cand_idx);
    return r;
}

template <typename T>
struct KeyOf;
template <>
struct KeyOf<float> {
    using U = uint32_t;
    static constexpr int BITS = 32;
    static constexpr int VEC = 4;  // elements of one 128-bit load
    static constexpr int PASSES = 3;
    __device__ static __forceinline__ U key(float v) {
        const U b = __float_as_uint(v + 0.0f);  // -0.0 + 0.0 = +0.0
        return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
    }
    __device__ static __forceinline__ float from_bits(uint32_t w0, uint32_t) { return __uint_as_float(w0); }
};
template <>
struct KeyOf<double> {
    using U = unsigned long long;
    static constexpr int BITS = 64;
    static constexpr int VEC = 2;
    static constexpr int PASSES = 6;
    __device__ static __forceinline__ U key(double v) {
        const U b = (U)__double_as_longlong(v + 0.0);
        return b ^ ((b >> 63) ? 0xFFFFFFFFFFFFFFFFull : 0x8000000000000000ull);
    }
    __device__ static __forceinline__ double from_bits(uint32_t w0, uint32_t w1) {
        return __longlong_as_double((long long)(((unsigned long long)w1 << 32) | w0));
    }
};

// Bits of digit `pass` and the shift that brings it to the bottom of the key.
template <typename T>
__host__ __device__ constexpr int topk_width(int pass) {
    return (KeyOf<T>::BITS == 32) ? (pass < 2 ? TOPK_WIDE : 10) : (pass < 4 ? TOPK_WIDE : 10);
}
template <typename T>
__host__ __device__ constexpr int topk_shift(int pass) {
    int s = KeyOf<T>::BITS;
    for (int p = 0; p <= pass; ++p) s -= topk_width<T>(p);
    return s;
}

__global__ __launch_bounds__(TOPK_WG) void topk_reset_kernel(TopkArgs a) {
    const TopkRow r = topk_row(a, blockIdx.x);
    for (int b = threadIdx.x; b < TOPK_MAX_BUCKETS; b += TOPK_WG) r.hist[b] = 0ull;
    if (threadIdx.x == 0) {
        r.st->prefix = 0ull;
        r.st->k_rem = a.k;
        r.st->n_out = 0ull;
        r.st->tie_min = ~0ull;
        r.st->ticket = 0u;
        r.st->overflow = 0u;
        r.st->cand_ok = 0u;
        r.st->n_ties = 0u;
    }
}

// Calls f(value, element index, valid) for the VEC elements of every aligned 128-bit vector
// that overlaps the row, the same number of times in every lane of the workgroup (so f may
// use wave-wide operations).  A vector that overlaps the row lies in one page with an element
// of the row, so reading all of it cannot fault; elements outside the row are flagged invalid.
template <typename T, typename F>
__device__ __forceinline__ void topk_for_each(const T* __restrict__ row_values, int64_t n, F&& f) {
    constexpr int VEC = KeyOf<T>::VEC;
    const int64_t lead = (int64_t)(((uintptr_t)row_values / sizeof(T)) % VEC);  // elements before the row
    const uint4* __restrict__ vecs = (const uint4*)(row_values - lead);
    const int64_t n_vec = (n + lead + VEC - 1) / VEC;
    const int64_t stride = (int64_t)gridDim.x * TOPK_WG;
    constexpr int FLIGHT = 4;  // 128-bit loads in flight per lane
    for (int64_t v0 = (int64_t)blockIdx.x * TOPK_WG; v0 < n_vec; v0 += FLIGHT * stride) {
        uint4 w[FLIGHT];
#pragma unroll
        for (int u = 0; u < FLIGHT; ++u) {
            const int64_t v = v0 + u * stride + threadIdx.x;
            w[u] = make_uint4(0, 0, 0, 0);
            if (v < n_vec) w[u] = vecs[v];
        }
#pragma unroll
        for (int u = 0; u < FLIGHT; ++u) {
            const int64_t v = v0 + u * stride + threadIdx.x;
            const bool in = v < n_vec;
            const uint32_t words[4] = {w[u].x, w[u].y, w[u].z, w[u].w};
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const int64_t e = v * VEC + j - lead;
                const T val = (VEC == 4) ? KeyOf<T>::from_bits(words[j], 0u)
                                         : KeyOf<T>::from_bits(words[(2 * j) & 3], words[(2 * j + 1) & 3]);
                f(val, e, in && e >= 0 && e < n);
            }
        }
    }
}

// Appends the flagged lanes' (key, index) pairs behind `*counter` with one atomic for the wave.
// Every lane of the wave must call it.  Slots at or beyond `cap` are dropped (the counter
// still counts them).
template <typename U>
__device__ __forceinline__ void topk_append(bool flag, U key, long long index, unsigned long long* counter,
                                            U* keys_out, long long* idx_out, unsigned long long cap) {
    const unsigned long long mask = __ballot(flag);
    if (mask == 0ull) return;
    const int lane = threadIdx.x & 63;
    unsigned long long base = 0ull;
    if (lane == 0) base = atomicAdd(counter, (unsigned long long)__popcll(mask));
    base = ((unsigned long long)__builtin_amdgcn_readfirstlane((int)(base >> 32)) << 32) |
           (unsigned int)__builtin_amdgcn_readfirstlane((int)(base & 0xFFFFFFFFull));
    if (flag) {
        const unsigned long long slot = base + (unsigned long long)__popcll(mask & ((1ull << lane) - 1ull));
        if (slot < cap) {
            keys_out[slot] = key;
            idx_out[slot] = index;
        }
    }
}

// One workgroup: walks the `1 << width` buckets from the top, fixes the digit that holds the
// k_rem-th largest matching key, and clears the histogram for the next pass.
__device__ __forceinline__ void topk_select_digit(TopkState* st, unsigned long long* hist, int width) {
    constexpr int PER = TOPK_MAX_BUCKETS / TOPK_WG;  // consecutive buckets per thread
    constexpr int WAVES = TOPK_WG / 64;
    __shared__ unsigned long long bins[TOPK_MAX_BUCKETS];
    __shared__ unsigned long long wave_sum[WAVES];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int n_buckets = 1 << width;
    // coalesced, independent loads (issued together), staged through LDS
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int b = t + TOPK_WG * j;
        bins[b] = b < n_buckets ? __hip_atomic_load(&hist[b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) hist[t + TOPK_WG * j] = 0ull;
    __syncthreads();
    unsigned long long h[PER];
    unsigned long long mine = 0ull;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        h[j] = bins[t * PER + j];
        mine += h[j];
    }
    // suffix sums over the threads: inside the wave by shuffles, across waves through LDS
    unsigned long long incl = mine;  // sum over lanes >= lane of this wave
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long o = __shfl_down(incl, off, 64);
        if (lane + off < 64) incl += o;
    }
    if (lane == 0) wave_sum[wave] = incl;
    __syncthreads();
    unsigned long long above = incl - mine;  // buckets of higher threads
    for (int w2 = wave + 1; w2 < WAVES; ++w2) above += wave_sum[w2];
    const unsigned long long k_rem = (unsigned long long)st->k_rem;
    const unsigned long long prefix = st->prefix;
    __syncthreads();
#pragma unroll
    for (int j = PER - 1; j >= 0; --j) {
        if (above < k_rem && k_rem <= above + h[j]) {
            st->prefix = (prefix << width) | (unsigned long long)(t * PER + j);
            st->k_rem = (long long)(k_rem - above);
        }
        above += h[j];
    }
}

// True in the workgroup of the row that arrives last; every workgroup calls it once per launch,
// after its own atomics on the row's state.  Waits until those have been performed.
__device__ __forceinline__ bool topk_last_workgroup(TopkState* st) {
    __shared__ unsigned int is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) is_last = (atomicAdd(&st->ticket, 1u) == gridDim.x - 1) ? 1u : 0u;
    __syncthreads();
    return is_last != 0u;
}

// Flushes the workgroup's LDS histogram, and lets the last workgroup of the row fix the digit.
// Returns true in that workgroup (after the selection).
__device__ __forceinline__ bool topk_finish_pass(TopkState* st, unsigned long long* hist, unsigned int* lh,
                                                 int width) {
    __syncthreads();
    for (int b = threadIdx.x; b < (1 << width); b += TOPK_WG) {
        const unsigned int c = lh[b];
        if (c) atomicAdd(&hist[b], (unsigned long long)c);
    }
    if (!topk_last_workgroup(st)) return false;
    topk_select_digit(st, hist, width);
    if (threadIdx.x == 0) st->ticket = 0u;
    return true;
}

// Pass 0: first digit of every key of the row.
template <typename T>
__global__ __launch_bounds__(TOPK_WG) void topk_first_kernel(const T* __restrict__ values, TopkArgs a) {
    using K = KeyOf<T>;
    __shared__ unsigned int lh[TOPK_MAX_BUCKETS];
    const TopkRow r = topk_row(a, blockIdx.y);
    constexpr int W = topk_width<T>(0), S = topk_shift<T>(0);
    for (int b = threadIdx.x; b < (1 << W); b += TOPK_WG) lh[b] = 0u;
    __syncthreads();
    topk_for_each<T>(values + (size_t)blockIdx.y * a.n, a.n, [&](T v, int64_t, bool valid) {
        if (valid) atomicAdd(&lh[(unsigned)(K::key(v) >> S)], 1u);
    });
    topk_finish_pass(r.st, r.hist, lh, W);
}

// Pass 1: winners above the first digit, candidates inside it, histogram of their second digit.
template <typename T>
__global__ __launch_bounds__(TOPK_WG) void topk_second_kernel(const T* __restrict__ values, TopkArgs a) {
    using K = KeyOf<T>;
    using U = typename K::U;
    __shared__ unsigned int lh[TOPK_MAX_BUCKETS];
    __shared__ unsigned int seg_count;
    const TopkRow r = topk_row(a, blockIdx.y);
    constexpr int W = topk_width<T>(1), S = topk_shift<T>(1), S0 = topk_shift<T>(0);
    for (int b = threadIdx.x; b < (1 << W); b += TOPK_WG) lh[b] = 0u;
    if (threadIdx.x == 0) seg_count = 0u;
    __syncthreads();
    const U first = (U)r.st->prefix;
    const int lane = threadIdx.x & 63;
    U* __restrict__ seg_keys = (U*)r.cand_keys + (size_t)blockIdx.x * a.seg_cap;
    long long* __restrict__ seg_idx = r.cand_idx + (size_t)blockIdx.x * a.seg_cap;
    topk_for_each<T>(values + (size_t)blockIdx.y * a.n, a.n, [&](T v, int64_t e, bool valid) {
        const U key = K::key(v);
        const U digit = key >> S0;
        const bool cand = valid && digit == first;
        topk_append(valid && digit > first, (unsigned long long)key, e, &r.st->n_out, r.keys, r.idx,
                    (unsigned long long)a.k);
        const unsigned long long mask = __ballot(cand);
        if (mask) {  // the wave's candidates go behind the workgroup's LDS counter
            unsigned int base = 0u;
            if (lane == 0) base = atomicAdd(&seg_count, (unsigned int)__popcll(mask));
            base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
            if (cand) {
                const unsigned int slot = base + (unsigned int)__popcll(mask & ((1ull << lane) - 1ull));
                if (slot < (unsigned int)a.seg_cap) {
                    seg_keys[slot] = key;
                    seg_idx[slot] = e;
                }
                atomicAdd(&lh[(unsigned)((key >> S) & ((1u << W) - 1u))], 1u);
            }
        }
    });
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int c = seg_count;
        r.counts[blockIdx.x] = c < (unsigned int)a.seg_cap ? c : (unsigned int)a.seg_cap;
        if (c > (unsigned int)a.seg_cap) atomicOr(&r.st->overflow, 1u);
    }
    if (topk_finish_pass(r.st, r.hist, lh, W) && threadIdx.x == 0)
        r.st->cand_ok = __hip_atomic_load(&r.st->overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ? 0u : 1u;
}

// Calls f(key, element index, valid) for every candidate of the row: from the side buffer, or
// from the row itself when the buffer was too small.  Uniform trip count per workgroup.
template <typename T, typename F>
__device__ __forceinline__ void topk_for_each_candidate(const T* __restrict__ row_values, const TopkArgs& a,
                                                        const TopkRow& r, F&& f) {
    using K = KeyOf<T>;
    using U = typename K::U;
    if (r.st->cand_ok) {
        const U* __restrict__ ck = (const U*)r.cand_keys;
        for (int seg = blockIdx.x; seg < a.n_seg; seg += gridDim.x) {
            const int count = (int)r.counts[seg];
            const size_t base = (size_t)seg * a.seg_cap;
            for (int i0 = 0; i0 < count; i0 += TOPK_WG) {
                const int i = i0 + threadIdx.x;
                const bool in = i < count;
                f(in ? ck[base + i] : (U)0, in ? r.cand_idx[base + i] : 0ll, in);
            }
        }
    } else {
        topk_for_each<T>(row_values, a.n, [&](T v, int64_t e, bool valid) { f(K::key(v), (long long)e, valid); });
    }
}

// Passes 2..: one more digit of the candidates that match the digits fixed so far.
template <typename T>
__global__ __launch_bounds__(TOPK_WG) void topk_next_kernel(const T* __restrict__ values, TopkArgs a, int width,
                                                            int shift) {
    using K = KeyOf<T>;
    using U = typename K::U;
    __shared__ unsigned int lh[TOPK_MAX_BUCKETS];
    const TopkRow r = topk_row(a, blockIdx.y);
    for (int b = threadIdx.x; b < (1 << width); b += TOPK_WG) lh[b] = 0u;
    __syncthreads();
    const U prefix = (U)r.st->prefix;
    const U digit_mask = (U)((1u << width) - 1u);
    topk_for_each_candidate<T>(values + (size_t)blockIdx.y * a.n, a, r, [&](U key, long long, bool valid) {
        if (valid && (key >> (shift + width)) == prefix) atomicAdd(&lh[(unsigned)((key >> shift) & digit_mask)], 1u);
    });
    topk_finish_pass(r.st, r.hist, lh, width);
}

// Candidates above the threshold key are winners; the lowest index holding the threshold key
// itself is tracked (the common case takes exactly one of them).  The last workgroup of the
// row then takes the k_rem lowest indices that hold the threshold key, walking the row in
// index order from the first of them and stopping as soon as it has enough.
template <typename T>
__global__ __launch_bounds__(TOPK_WG) void topk_gather_kernel(const T* __restrict__ values, TopkArgs a) {
    using K = KeyOf<T>;
    using U = typename K::U;
    const TopkRow r = topk_row(a, blockIdx.y);
    const T* __restrict__ row_values = values + (size_t)blockIdx.y * a.n;
    constexpr int S0 = topk_shift<T>(0);
    const U thr = (U)r.st->prefix;
    const U first = thr >> S0;
    const int lane = threadIdx.x & 63;
    long long* __restrict__ tie_list = (long long*)r.hist;
    __shared__ unsigned int ties_full;
    if (threadIdx.x == 0) ties_full = 0u;
    __syncthreads();
    topk_for_each_candidate<T>(row_values, a, r, [&](U key, long long e, bool valid) {
        const bool mine = valid && (key >> S0) == first;  // keys above the first digit went out in pass 1
        topk_append<unsigned long long>(mine && key > thr, (unsigned long long)key, e, &r.st->n_out, r.keys, r.idx,
                                        (unsigned long long)a.k);
        const bool tie = mine && key == thr;
        const unsigned long long tie_mask = __ballot(tie);
        if (tie_mask) {
            unsigned long long m = tie ? (unsigned long long)e : ~0ull;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const unsigned long long o = __shfl_xor(m, off, 64);
                m = o < m ? o : m;
            }
            if (lane == 0) atomicMin(&r.st->tie_min, m);
            // the indices that hold the threshold key are listed in the (now unused) histogram
            // while they fit; a workgroup stops once it has seen the list full
            if (!ties_full) {
                unsigned int base = 0u;
                if (lane == 0) base = atomicAdd(&r.st->n_ties, (unsigned int)__popcll(tie_mask));
                base = (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
                if (tie) {
                    const unsigned int slot = base + (unsigned int)__popcll(tie_mask & ((1ull << lane) - 1ull));
                    if (slot < TOPK_TIE_LIST)  // read by another workgroup of this launch: device-scope store
                        __hip_atomic_store(&tie_list[slot], e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (base + (unsigned int)__popcll(tie_mask) > TOPK_TIE_LIST) ties_full = 1u;  // benign race
            }
        }
    });

    if (!topk_last_workgroup(r.st)) return;
    const long long k_rem = r.st->k_rem;
    const long long base_slot = (long long)a.k - k_rem;
    const unsigned long long tie_min =
        __hip_atomic_load(&r.st->tie_min, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x == 0) r.st->ticket = 0u;
    if (k_rem == 1) {
        if (threadIdx.x == 0) {
            r.keys[base_slot] = (unsigned long long)thr;
            r.idx[base_slot] = (long long)tie_min;
        }
        return;
    }
    const unsigned int n_ties = __hip_atomic_load(&r.st->n_ties, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (n_ties <= TOPK_TIE_LIST) {
        // the list is complete: its k_rem lowest indices, by rank
        __shared__ long long ties[TOPK_TIE_LIST];
        for (unsigned int i = threadIdx.x; i < n_ties; i += TOPK_WG)
            ties[i] = (long long)__hip_atomic_load((unsigned long long*)&tie_list[i], __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        for (unsigned int i = threadIdx.x; i < n_ties; i += TOPK_WG) {
            const long long mine = ties[i];
            long long rank = 0;
            for (unsigned int j = 0; j < n_ties; ++j) rank += ties[j] < mine ? 1 : 0;
            if (rank < k_rem) {
                r.keys[base_slot + rank] = (unsigned long long)thr;
                r.idx[base_slot + rank] = mine;
            }
        }
        return;
    }
    // too many to list: they are dense, and walking the row in index order from the first of
    // them finds k_rem of them soon
    __shared__ int wave_counts[TOPK_WG / 64];
    __shared__ long long taken_s;
    if (threadIdx.x == 0) taken_s = 0;
    __syncthreads();
    const int wave = threadIdx.x >> 6;
    for (int64_t i0 = (int64_t)tie_min; i0 < a.n; i0 += TOPK_WG) {
        const long long taken = taken_s;
        if (taken >= k_rem) break;
        const int64_t i = i0 + threadIdx.x;
        const bool flag = (i < a.n) && (K::key(row_values[i]) == thr);
        const unsigned long long mask = __ballot(flag);
        if (lane == 0) wave_counts[wave] = __popcll(mask);
        __syncthreads();
        long long offset = taken;
        int all = 0;
        for (int w2 = 0; w2 < TOPK_WG / 64; ++w2) {
            if (w2 < wave) offset += wave_counts[w2];
            all += wave_counts[w2];
        }
        const long long rank = offset + __popcll(mask & ((1ull << lane) - 1ull));
        if (flag && rank < k_rem) {
            r.keys[base_slot + rank] = (unsigned long long)thr;
            r.idx[base_slot + rank] = i;
        }
        __syncthreads();
        if (threadIdx.x == 0) taken_s = taken + all;
        __syncthreads();
    }
}

// Rank sort of the k winners of a row (descending key, ascending index); writes the indices
// and/or the values in that order.
template <typename T>
__global__ __launch_bounds__(256) void topk_order_kernel(const T* __restrict__ values, TopkArgs a,
                                                         int64_t* __restrict__ out_idx, T* __restrict__ out_values) {
    const TopkRow r = topk_row(a, blockIdx.y);
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= a.k) return;
    const unsigned long long ki = r.keys[i];
    const long long ii = r.idx[i];
    int rank = 0;
    for (int j = 0; j < a.k; ++j) {
        const unsigned long long kj = r.keys[j];
        const long long ij = r.idx[j];
        rank += (kj > ki || (kj == ki && ij < ii)) ? 1 : 0;
    }
    const size_t o = (size_t)blockIdx.y * a.k + rank;
    if (out_idx) out_idx[o] = ii;
    if (out_values) out_values[o] = values[(size_t)blockIdx.y * a.n + ii];
}

// ------------------------------------------------------------------------------------------
// Small k on one row of moderate length: ONE read of the row and two launches.
//
// Every element is an item (key, index), ordered by descending key, then ascending index: no two
// items are equal, so "the k largest" needs no rule for ties.  A workgroup of 1024 threads takes
// VPT elements per thread into registers.  The k-th largest of the 1024 THREAD MAXIMA (a radix
// select over their bytes, a histogram of 256 bins in LDS per byte) is a threshold that at least
// k items reach and that at most k threads have an item above: the items that reach it - at most
// k VPT - are collected in LDS and ranked against each other, and those of rank below k are the
// workgroup's k largest, in order.  A second launch of one workgroup does the same with the
// workgroups' results and writes the answer.
constexpr int TOPK_SMALL_K = 64;       // largest k of this path
constexpr int TOPK_SMALL_CAND = 2048;  // items the ranking step holds (k * items per thread at most)
constexpr int TOPK_SMALL_WGS = 1024;   // workgroups of the first launch at most

template <typename T>
struct SmallItem {
    typename KeyOf<T>::U key;  // 0: no item (every real key is above it)
    uint32_t idx;
};
template <typename T>
__device__ __forceinline__ bool item_gt(const SmallItem<T>& a, const SmallItem<T>& b) {
    return a.key > b.key || (a.key == b.key && a.idx < b.idx);
}

// The k largest of the workgroup's items (NV per thread, in registers), written in order to
// top_key / top_idx (k entries, no-item fillers at the end when there are fewer).  Every thread
// of the 1024 calls it.
template <typename T, int NV>
__device__ inline void small_topk_of_workgroup(const SmallItem<T> (&items)[NV], int k,
                                               typename KeyOf<T>::U* __restrict__ top_key,
                                               uint32_t* __restrict__ top_idx) {
    using U = typename KeyOf<T>::U;
    constexpr int KEY_BYTES = (int)sizeof(U), PASSES = KEY_BYTES + 4;
    __shared__ unsigned int hist[256];
    __shared__ unsigned int sel_digit, sel_rem, n_cand, n_valid;
    __shared__ U cand_key[TOPK_SMALL_CAND];
    __shared__ uint32_t cand_idx[TOPK_SMALL_CAND];
    SmallItem<T> best = items[0];
#pragma unroll
    for (int v = 1; v < NV; ++v)
        if (item_gt<T>(items[v], best)) best = items[v];
    if (threadIdx.x < 256) hist[threadIdx.x] = 0u;
    if (threadIdx.x == 0) {
        n_cand = 0u;
        n_valid = 0u;
        sel_rem = 0u;
    }
    __syncthreads();
    const unsigned long long has = __ballot(best.key != 0);
    if ((threadIdx.x & 63) == 0 && has) atomicAdd(&n_valid, (unsigned int)__popcll(has));
    __syncthreads();
    // threshold: the k-th largest thread maximum, byte by byte from the top (key, then inverted
    // index); with at most k maxima every item passes
    SmallItem<T> thr;
    thr.key = 0;
    thr.idx = 0xffffffffu;
    if (n_valid > (unsigned int)k) {
        bool alive = best.key != 0;
        unsigned int rem = (unsigned int)k;  // the threshold is the rem-th largest of the maxima still alive
        U pk = 0;
        uint32_t pi = 0;  // (of the inverted index)
        for (int p = 0; p < PASSES; ++p) {
            const unsigned int digit = p < KEY_BYTES ? (unsigned int)(best.key >> (8 * (KEY_BYTES - 1 - p))) & 255u
                                                     : ((~best.idx) >> (8 * (PASSES - 1 - p))) & 255u;
            if (alive) atomicAdd(&hist[digit], 1u);
            __syncthreads();
            if (threadIdx.x < 64) {
                // lane l: the bins 4 l .. 4 l + 3; the bin in which the count from the top reaches rem
                const unsigned int b0 = hist[4 * threadIdx.x], b1 = hist[4 * threadIdx.x + 1],
                                   b2 = hist[4 * threadIdx.x + 2], b3 = hist[4 * threadIdx.x + 3];
                const unsigned int mine = b0 + b1 + b2 + b3;
                // count in the bins of the higher lanes: an inclusive suffix sum over the lanes, by doubling
                unsigned int suffix = mine;
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) {
                    const unsigned int o = __shfl_down(suffix, off, 64);
                    if ((int)threadIdx.x + off < 64) suffix += o;
                }
                const unsigned int above = suffix - mine;
                if (above < rem && rem <= above + mine) {
                    unsigned int acc = above, d = 4 * threadIdx.x + 3, left = rem;
                    const unsigned int bins[4] = {b3, b2, b1, b0};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (acc < rem && rem <= acc + bins[j]) {
                            d = 4 * threadIdx.x + 3 - j;
                            left = rem - acc;
                        }
                        acc += bins[j];
                    }
                    sel_digit = d;
                    sel_rem = left;
                }
            }
            __syncthreads();
            const unsigned int sd = sel_digit;
            rem = sel_rem;
            alive = alive && digit == sd;
            if (p < KEY_BYTES)
                pk |= (U)sd << (8 * (KEY_BYTES - 1 - p));
            else
                pi |= sd << (8 * (PASSES - 1 - p));
            if (threadIdx.x < 256) hist[threadIdx.x] = 0u;
            __syncthreads();
        }
        thr.key = pk;
        thr.idx = ~pi;
    }
    // the items that reach the threshold
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        if (items[v].key != 0 && !item_gt<T>(thr, items[v])) {
            const unsigned int at = atomicAdd(&n_cand, 1u);
            if (at < (unsigned int)TOPK_SMALL_CAND) {
                cand_key[at] = items[v].key;
                cand_idx[at] = items[v].idx;
            }
        }
    }
    __syncthreads();
    const int nc = (int)min(n_cand, (unsigned int)TOPK_SMALL_CAND);
    for (int j = nc + (int)threadIdx.x; j < k; j += blockDim.x) {  // (fewer items than k: fillers at the end)
        top_key[j] = 0;
        top_idx[j] = 0xffffffffu;
    }
    for (int c = threadIdx.x; c < nc; c += blockDim.x) {
        SmallItem<T> me;
        me.key = cand_key[c];
        me.idx = cand_idx[c];
        int rank = 0;
        for (int j = 0; j < nc; ++j) {
            SmallItem<T> o;
            o.key = cand_key[j];
            o.idx = cand_idx[j];
            rank += item_gt<T>(o, me) ? 1 : 0;
        }
        if (rank < k) {
            top_key[rank] = me.key;
            top_idx[rank] = me.idx;
        }
    }
}

template <typename T, int VPT>
__global__ __launch_bounds__(TOPK_WG) void topk_small_partial_kernel(const T* __restrict__ values, int64_t n, int k,
                                                                     typename KeyOf<T>::U* __restrict__ part_key,
                                                                     uint32_t* __restrict__ part_idx, int vec_ok) {
    constexpr int VEC = KeyOf<T>::VEC, NL = VPT / VEC;  // 128-bit loads per thread
    SmallItem<T> items[VPT];
    const int64_t base = (int64_t)blockIdx.x * (TOPK_WG * VPT);
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int64_t i0 = base + ((int64_t)j * TOPK_WG + threadIdx.x) * VEC;
        T v[VEC];
        if (vec_ok && i0 + VEC <= n) {
            const uint4 q = *reinterpret_cast<const uint4*>(values + i0);
            if (VEC == 4) {
                v[0] = KeyOf<T>::from_bits(q.x, 0);
                v[1] = KeyOf<T>::from_bits(q.y, 0);
                v[VEC - 2] = KeyOf<T>::from_bits(q.z, 0);
                v[VEC - 1] = KeyOf<T>::from_bits(q.w, 0);
            } else {
                v[0] = KeyOf<T>::from_bits(q.x, q.y);
                v[VEC - 1] = KeyOf<T>::from_bits(q.z, q.w);
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = i0 + e < n ? values[i0 + e] : T(0);
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            items[j * VEC + e].key = i0 + e < n ? KeyOf<T>::key(v[e]) : 0;
            items[j * VEC + e].idx = (uint32_t)(i0 + e);
        }
    }
    small_topk_of_workgroup<T, VPT>(items, k, part_key + (size_t)blockIdx.x * k, part_idx + (size_t)blockIdx.x * k);
}

template <typename T, int IPT>
__global__ __launch_bounds__(TOPK_WG) void topk_small_merge_kernel(const T* __restrict__ values, int n_items, int k,
                                                                   const typename KeyOf<T>::U* __restrict__ part_key,
                                                                   const uint32_t* __restrict__ part_idx,
                                                                   int64_t* __restrict__ out_idx,
                                                                   T* __restrict__ out_values) {
    using U = typename KeyOf<T>::U;
    __shared__ U top_key[TOPK_SMALL_K];
    __shared__ uint32_t top_idx[TOPK_SMALL_K];
    SmallItem<T> items[IPT];
#pragma unroll
    for (int v = 0; v < IPT; ++v) {
        const int i = v * TOPK_WG + (int)threadIdx.x;
        items[v].key = i < n_items ? part_key[i] : 0;
        items[v].idx = i < n_items ? part_idx[i] : 0xffffffffu;
    }
    small_topk_of_workgroup<T, IPT>(items, k, top_key, top_idx);
    __syncthreads();
    for (int j = threadIdx.x; j < k; j += TOPK_WG) {
        if (top_key[j] != 0) {  // (k <= n: every slot is filled)
            if (out_idx) out_idx[j] = (int64_t)top_idx[j];
            if (out_values) out_values[j] = values[top_idx[j]];
        }
    }
}

// Elements per thread of the first launch (0: the row is not for this path).
template <typename T>
int topk_small_vpt(int64_t rows, int64_t n, int32_t k) {
    if (rows != 1 || k > TOPK_SMALL_K || n >= ((int64_t)1 << 32) - 1) return 0;
    constexpr int VEC = KeyOf<T>::VEC;
    for (int vpt = VEC; vpt <= 16; vpt *= 2) {
        const int64_t g = kmx_cdiv(n, (int64_t)TOPK_WG * vpt);
        // (few workgroups while the row is short, never more than the second launch can take)
        if ((g <= 256 || vpt == 16) && g <= TOPK_SMALL_WGS && g * k <= 32 * TOPK_WG && (int64_t)k * vpt <= TOPK_SMALL_CAND)
            return vpt;
    }
    return 0;
}

template <typename T>
int32_t topk_small_impl(const T* values, int64_t* out_idx, T* out_values, int64_t n, int32_t k, char* area, int vpt,
                        hipStream_t stream) {
    using U = typename KeyOf<T>::U;
    const int g = (int)kmx_cdiv(n, (int64_t)TOPK_WG * vpt);
    U* part_key = reinterpret_cast<U*>(area);
    uint32_t* part_idx = reinterpret_cast<uint32_t*>(area + kmx_align256((size_t)g * k * sizeof(U)));
    const int vec_ok = (((uintptr_t)values) & 15) == 0;
#define KMX_TOPK_PART(VPT_)                                                                                     \
    hipLaunchKernelGGL((topk_small_partial_kernel<T, VPT_>), dim3((unsigned)g), dim3(TOPK_WG), 0, stream, values, n, \
                       (int)k, part_key, part_idx, vec_ok)
    if constexpr (KeyOf<T>::VEC == 2) {
        if (vpt == 2) KMX_TOPK_PART(2);
    }
    if (vpt == 4) KMX_TOPK_PART(4);
    else if (vpt == 8) KMX_TOPK_PART(8);
    else if (vpt == 16) KMX_TOPK_PART(16);
#undef KMX_TOPK_PART
    const int n_items = g * k;
    const int ipt = (int)kmx_cdiv(n_items, TOPK_WG);
#define KMX_TOPK_MERGE(IPT_)                                                                                  \
    hipLaunchKernelGGL((topk_small_merge_kernel<T, IPT_>), dim3(1), dim3(TOPK_WG), 0, stream, values, n_items, \
                       (int)k, part_key, part_idx, out_idx, out_values)
    if (ipt <= 1) KMX_TOPK_MERGE(1);
    else if (ipt <= 2) KMX_TOPK_MERGE(2);
    else if (ipt <= 4) KMX_TOPK_MERGE(4);
    else if (ipt <= 8) KMX_TOPK_MERGE(8);
    else if (ipt <= 16) KMX_TOPK_MERGE(16);
    else KMX_TOPK_MERGE(32);
#undef KMX_TOPK_MERGE
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// bytes of the first launch's results (the largest grid, the wider key)
size_t topk_small_bytes(int64_t n, int32_t k) {
    if (k > TOPK_SMALL_K) return 0;
    const int64_t g = kmx_cdiv(n, (int64_t)TOPK_WG * 2) < TOPK_SMALL_WGS ? kmx_cdiv(n, (int64_t)TOPK_WG * 2) : TOPK_SMALL_WGS;
    return kmx_align256((size_t)g * k * 8) + kmx_align256((size_t)g * k * 4);
}

template <typename T>
int32_t topk_impl(const void* values_, int64_t* out_idx, void* out_values, int64_t rows, int64_t n, int32_t k,
                  char* ws, int32_t dtype, hipStream_t stream) {
    const TopkLayout L = topk_layout(rows, n, k, dtype);
    if (const int vpt = topk_small_vpt<T>(rows, n, k); vpt != 0)
        return topk_small_impl<T>((const T*)values_, out_idx, (T*)out_values, n, k, ws + L.off_small, vpt, stream);
    // rows are taken in slices of the grid's second dimension
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
        const int64_t nr = rows - r0 < 65535 ? rows - r0 : 65535;
        const T* values = (const T*)values_ + (size_t)r0 * n;
        TopkArgs a;
        a.ws = ws + (size_t)r0 * L.row_bytes;
        a.row_bytes = L.row_bytes;
        a.off_hist = L.off_hist;
        a.off_counts = L.off_counts;
        a.off_keys = L.off_keys;
        a.off_idx = L.off_idx;
        a.off_cand_keys = L.off_cand_keys;
        a.off_cand_idx = L.off_cand_idx;
        a.n = n;
        a.k = k;
        a.n_seg = (int32_t)L.n_seg;
        a.seg_cap = (int32_t)L.seg_cap;
        // the passes over the candidates: a quarter of the workgroups (each takes several segments)
        const int64_t per_row_cand = L.n_seg >= 4 ? L.n_seg / 4 : 1;
        const dim3 grid_full((unsigned)L.n_seg, (unsigned)nr), grid_cand((unsigned)per_row_cand, (unsigned)nr);
        hipLaunchKernelGGL(topk_reset_kernel, dim3((unsigned)nr), dim3(TOPK_WG), 0, stream, a);
        hipLaunchKernelGGL((topk_first_kernel<T>), grid_full, dim3(TOPK_WG), 0, stream, values, a);
        hipLaunchKernelGGL((topk_second_kernel<T>), grid_full, dim3(TOPK_WG), 0, stream, values, a);
        for (int p = 2; p < KeyOf<T>::PASSES; ++p)
            hipLaunchKernelGGL((topk_next_kernel<T>), grid_cand, dim3(TOPK_WG), 0, stream, values, a,
                               topk_width<T>(p), topk_shift<T>(p));
        hipLaunchKernelGGL((topk_gather_kernel<T>), grid_cand, dim3(TOPK_WG), 0, stream, values, a);
        hipLaunchKernelGGL((topk_order_kernel<T>), dim3((unsigned)kmx_cdiv(k, 256), (unsigned)nr), dim3(256), 0,
                           stream, values, a, out_idx ? out_idx + (size_t)r0 * k : nullptr,
                           out_values ? (T*)out_values + (size_t)r0 * k : nullptr);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t topk_entry(const void* values, int64_t* out_idx, void* out_values, int64_t rows, int64_t n, int32_t k,
                   void* workspace, size_t workspace_bytes, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(values);
    KMX_REQUIRE_PTR(workspace);
    if (rows <= 0 || n <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    if (k > n) return KMX_ERR_BAD_ARGUMENT;
    KMX_REQUIRE_DTYPE(dtype);
    if (workspace_bytes < kmx_topk_rows_workspace_bytes(rows, n, k, dtype)) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        return topk_impl<float>(values, out_idx, out_values, rows, n, k, (char*)workspace, dtype, stream);
    return topk_impl<double>(values, out_idx, out_values, rows, n, k, (char*)workspace, dtype, stream);
}

}  // namespace

extern "C" {

size_t kmx_topk_rows_workspace_bytes(int64_t rows, int64_t n, int32_t k, int32_t dtype) {
    if (rows <= 0 || n <= 0 || k <= 0 || k > n) return 0;
    if (dtype != KMX_F32 && dtype != KMX_F64) return 0;
    return (size_t)rows * topk_layout(rows, n, k, dtype).row_bytes;
}

size_t kmx_topk_workspace_bytes(int64_t n, int32_t k) { return kmx_topk_rows_workspace_bytes(1, n, k, KMX_F64); }

int32_t kmx_topk_idx_rows(const void* values, int64_t* out_indices, int64_t rows, int64_t n, int32_t k,
                          void* workspace, size_t workspace_bytes, int32_t dtype, void* stream) {
    KMX_REQUIRE_PTR(out_indices);
    return topk_entry(values, out_indices, nullptr, rows, n, k, workspace, workspace_bytes, dtype, stream);
}

int32_t kmx_topk_values(const void* values, void* out_values, int64_t rows, int64_t n, int32_t k, void* workspace,
                        size_t workspace_bytes, int32_t dtype, void* stream) {
    KMX_REQUIRE_PTR(out_values);
    return topk_entry(values, nullptr, out_values, rows, n, k, workspace, workspace_bytes, dtype, stream);
}

int32_t kmx_topk_idx(const void* values, int64_t* out_indices, int64_t n, int32_t k, void* workspace,
                     size_t workspace_bytes, int32_t dtype, void* stream) {
    KMX_REQUIRE_PTR(out_indices);
    return topk_entry(values, out_indices, nullptr, 1, n, k, workspace, workspace_bytes, dtype, stream);
}

}  // extern "C"
