// Radix-select top-k of a 1-D float array on gfx950 (used to relocate empty clusters onto
// the samples farthest from their centroid).
//
// Floats are mapped to unsigned keys whose integer order is the float order.  The key of the
// k-th largest value is fixed 8 bits at a time, most significant digit first: each pass
// histograms one digit of the keys that match the prefix found so far (LDS histogram per
// workgroup, flushed with 64-bit atomics), then a one-workgroup kernel walks the 256 buckets
// from the top.  4 passes for fp32, 8 for fp64; nothing returns to the host in between.
// Selection afterwards: every key above the threshold, plus the needed number of keys equal
// to it, lowest indices first.  The k winners are finally ordered by descending value, then
// ascending index, so the result is deterministic.
#include "kmx_common.h"

namespace {

struct TopkState {
    unsigned long long prefix;      // digits fixed so far (threshold key after the last pass)
    long long k_rem;                // how many keys equal to the threshold belong to the top k
    unsigned long long n_greater;   // slot counter of the gather
    unsigned long long tie_min;     // lowest index holding the threshold key
    unsigned long long n_ties_taken;
    unsigned long long pad[3];
};

struct TopkLayout {
    size_t off_state, off_hist, off_keys, off_idx, total;
};

TopkLayout topk_layout(int32_t k) {
    TopkLayout L;
    L.off_state = 0;
    L.off_hist = 256;
    L.off_keys = L.off_hist + 256 * sizeof(unsigned long long);
    L.off_idx = L.off_keys + kmx_align256((size_t)k * sizeof(unsigned long long));
    L.total = L.off_idx + kmx_align256((size_t)k * sizeof(long long));
    return L;
}

template <typename T>
struct KeyOf;
template <>
struct KeyOf<float> {
    using U = uint32_t;
    static constexpr int BITS = 32;
    __device__ static __forceinline__ U key(float v) {
        const U b = __float_as_uint(v);
        return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
    }
};
template <>
struct KeyOf<double> {
    using U = unsigned long long;
    static constexpr int BITS = 64;
    __device__ static __forceinline__ U key(double v) {
        const U b = (U)__double_as_longlong(v);
        return b ^ ((b >> 63) ? 0xFFFFFFFFFFFFFFFFull : 0x8000000000000000ull);
    }
};

__global__ void topk_reset_kernel(TopkState* st, unsigned long long* hist, int32_t k) {
    hist[threadIdx.x] = 0ull;
    if (threadIdx.x == 0) {
        st->prefix = 0ull;
        st->k_rem = k;
        st->n_greater = 0ull;
        st->tie_min = ~0ull;
        st->n_ties_taken = 0ull;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void topk_hist_kernel(const T* __restrict__ values, int64_t n,
                                                        const TopkState* __restrict__ st,
                                                        unsigned long long* __restrict__ hist,
                                                        int pass) {
    using K = KeyOf<T>;
    using U = typename K::U;
    __shared__ unsigned int lh[256];
    lh[threadIdx.x] = 0u;
    __syncthreads();
    const int shift = K::BITS - 8 * (pass + 1);
    const U prefix = (U)st->prefix;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const U key = K::key(values[i]);
        const bool match = (pass == 0) || ((key >> (shift + 8)) == prefix);
        if (match) atomicAdd(&lh[(unsigned)((key >> shift) & 0xFF)], 1u);
    }
    __syncthreads();
    const unsigned int c = lh[threadIdx.x];
    if (c) atomicAdd(&hist[threadIdx.x], (unsigned long long)c);
}

// One workgroup of 256 threads, thread b = bucket b.
__global__ __launch_bounds__(256) void topk_select_kernel(TopkState* st, unsigned long long* hist) {
    __shared__ unsigned long long suffix[257];
    const int b = threadIdx.x;
    const unsigned long long h = hist[b];
    suffix[b] = h;
    if (b == 0) suffix[256] = 0ull;
    __syncthreads();
    // inclusive suffix sums: suffix[b] = sum_{b' >= b} h[b']
    for (int off = 1; off < 256; off <<= 1) {
        unsigned long long add = 0ull;
        if (b + off < 256) add = suffix[b + off];
        __syncthreads();
        suffix[b] += add;
        __syncthreads();
    }
    const unsigned long long k_rem = (unsigned long long)st->k_rem;
    const unsigned long long above = suffix[b + 1];
    __syncthreads();
    if (above < k_rem && k_rem <= above + h) {
        st->prefix = (st->prefix << 8) | (unsigned long long)b;
        st->k_rem = (long long)(k_rem - above);
    }
    hist[b] = 0ull;
}

// Keys strictly above the threshold go to free slots (order fixed later); the lowest index
// holding the threshold itself is tracked for the common single-tie case.
template <typename T>
__global__ __launch_bounds__(256) void topk_gather_kernel(const T* __restrict__ values, int64_t n,
                                                          TopkState* __restrict__ st,
                                                          unsigned long long* __restrict__ keys,
                                                          long long* __restrict__ idx) {
    using K = KeyOf<T>;
    using U = typename K::U;
    const U thr = (U)st->prefix;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const U key = K::key(values[i]);
        if (key > thr) {
            const unsigned long long slot = atomicAdd(&st->n_greater, 1ull);
            keys[slot] = (unsigned long long)key;
            idx[slot] = i;
        } else if (key == thr) {
            atomicMin(&st->tie_min, (unsigned long long)i);
        }
    }
}

// Takes the k_rem lowest indices holding the threshold key.  One workgroup walks the array in
// index order and stops as soon as enough ties are found.
template <typename T>
__global__ __launch_bounds__(1024) void topk_ties_kernel(const T* __restrict__ values, int64_t n,
                                                         TopkState* __restrict__ st,
                                                         unsigned long long* __restrict__ keys,
                                                         long long* __restrict__ idx, int32_t k) {
    using K = KeyOf<T>;
    using U = typename K::U;
    const U thr = (U)st->prefix;
    const long long k_rem = st->k_rem;
    const long long base_slot = (long long)k - k_rem;
    if (k_rem == 1) {
        if (threadIdx.x == 0) {
            keys[base_slot] = (unsigned long long)thr;
            idx[base_slot] = (long long)st->tie_min;
        }
        return;
    }
    __shared__ int wave_counts[16];
    __shared__ long long taken_s;
    if (threadIdx.x == 0) taken_s = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int64_t i0 = st->tie_min; i0 < n; i0 += 1024) {
        const long long taken = taken_s;
        if (taken >= k_rem) break;
        const int64_t i = i0 + threadIdx.x;
        const bool flag = (i < n) && (K::key(values[i]) == thr);
        const unsigned long long mask = __ballot(flag);
        if (lane == 0) wave_counts[wave] = __popcll(mask);
        __syncthreads();
        long long offset = taken;
        int all = 0;
        for (int w2 = 0; w2 < 16; ++w2) {
            if (w2 < wave) offset += wave_counts[w2];
            all += wave_counts[w2];
        }
        const long long rank = offset + __popcll(mask & ((1ull << lane) - 1ull));
        if (flag && rank < k_rem) {
            keys[base_slot + rank] = (unsigned long long)thr;
            idx[base_slot + rank] = i;
        }
        __syncthreads();
        if (threadIdx.x == 0) taken_s = taken + all;
        __syncthreads();
    }
}

// Rank sort of the k winners: descending key, ascending index.
__global__ __launch_bounds__(256) void topk_order_kernel(const unsigned long long* __restrict__ keys,
                                                         const long long* __restrict__ idx,
                                                         int64_t* __restrict__ out, int32_t k) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= k) return;
    const unsigned long long ki = keys[i];
    const long long ii = idx[i];
    int rank = 0;
    for (int j = 0; j < k; ++j) {
        const unsigned long long kj = keys[j];
        const long long ij = idx[j];
        rank += (kj > ki || (kj == ki && ij < ii)) ? 1 : 0;
    }
    out[rank] = ii;
}

template <typename T>
int32_t topk_impl(const void* values, int64_t* out, int64_t n, int32_t k, char* ws,
                  hipStream_t stream) {
    const TopkLayout L = topk_layout(k);
    auto* st = (TopkState*)(ws + L.off_state);
    auto* hist = (unsigned long long*)(ws + L.off_hist);
    auto* keys = (unsigned long long*)(ws + L.off_keys);
    auto* idx = (long long*)(ws + L.off_idx);
    int64_t blocks = kmx_cdiv(n, 256 * 8);
    const int64_t cap = (int64_t)kmx_num_cus() * 4;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(topk_reset_kernel, dim3(1), dim3(256), 0, stream, st, hist, k);
    const int passes = KeyOf<T>::BITS / 8;
    for (int p = 0; p < passes; ++p) {
        hipLaunchKernelGGL((topk_hist_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                           (const T*)values, n, st, hist, p);
        hipLaunchKernelGGL(topk_select_kernel, dim3(1), dim3(256), 0, stream, st, hist);
    }
    hipLaunchKernelGGL((topk_gather_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const T*)values, n, st, keys, idx);
    hipLaunchKernelGGL((topk_ties_kernel<T>), dim3(1), dim3(1024), 0, stream, (const T*)values, n,
                       st, keys, idx, k);
    hipLaunchKernelGGL(topk_order_kernel, dim3((unsigned)kmx_cdiv(k, 256)), dim3(256), 0, stream,
                       keys, idx, out, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

}  // namespace

extern "C" {

size_t kmx_topk_workspace_bytes(int64_t n, int32_t k) {
    if (n <= 0 || k <= 0 || k > n) return 0;
    return topk_layout(k).total;
}

int32_t kmx_topk_idx(const void* values, int64_t* out_indices, int64_t n, int32_t k,
                     void* workspace, size_t workspace_bytes, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(values);
    KMX_REQUIRE_PTR(out_indices);
    KMX_REQUIRE_PTR(workspace);
    if (n <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    if (k > n) return KMX_ERR_BAD_ARGUMENT;
    KMX_REQUIRE_DTYPE(dtype);
    if (workspace_bytes < topk_layout(k).total) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32) return topk_impl<float>(values, out_indices, n, k, (char*)workspace, stream);
    return topk_impl<double>(values, out_indices, n, k, (char*)workspace, stream);
}

}  // extern "C"
