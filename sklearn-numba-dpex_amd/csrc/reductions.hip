// Shared reduction and elementwise kernels for gfx950 (the reference's common/ kernels):
// row/column sums, argmin, half squared norms, broadcast ops, label bookkeeping.
// Sums accumulate in fp64 in a fixed order (thread-strided, wave shuffle tree, wave order,
// block order), so results do not change from run to run.
#include "kmx_common.h"

#include <atomic>
#include <mutex>
#include <type_traits>

namespace {

constexpr int SUM_MAX_BLOCKS_PER_ROW = 256;
constexpr int SUM_COL_CHUNKS = 64;

// VEC: rows start 16-byte aligned and hold a whole number of 16-byte groups; a thread then
// reads 16 bytes per load and keeps two loads in flight.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sum_rows_stage1(const T* __restrict__ in,
                                                       double* __restrict__ partial, int64_t cols,
                                                       int square) {
    const int64_t row = blockIdx.y;
    const T* __restrict__ p = in + (size_t)row * cols;
    double acc = 0.0;
    if constexpr (VEC) {
        constexpr int W = 16 / sizeof(T);
        using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
        const V* __restrict__ pv = reinterpret_cast<const V*>(p);
        const int64_t groups = cols / W;
        const int64_t stride = (int64_t)gridDim.x * 256;
        int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
        auto add = [&](const V& v) {
            const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                const double x = (double)e[j];
                acc += square ? x * x : x;
            }
        };
        for (; g + stride < groups; g += 2 * stride) {
            const V a = pv[g];
            const V b = pv[g + stride];
            add(a);
            add(b);
        }
        if (g < groups) add(pv[g]);
    } else {
        const int64_t stride = (int64_t)gridDim.x * 256;
        for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += stride) {
            const double v = (double)p[c];
            acc += square ? v * v : v;
        }
    }
    __shared__ double scratch[4];
    const double tot = kmx_block_sum<double>(acc, scratch);
    if (threadIdx.x == 0) partial[(size_t)row * gridDim.x + blockIdx.x] = tot;
}

template <typename T>
__global__ __launch_bounds__(256) void sum_rows_stage2(const double* __restrict__ partial,
                                                       T* __restrict__ out, int n_partials) {
    const int64_t row = blockIdx.x;
    double acc = 0.0;
    for (int j = threadIdx.x; j < n_partials; j += 256) acc += partial[(size_t)row * n_partials + j];
    __shared__ double scratch[4];
    const double tot = kmx_block_sum<double>(acc, scratch);
    if (threadIdx.x == 0) out[row] = (T)tot;
}

// Row sums in ONE launch (up to SUM_TICKET_ROWS rows): stage 1 as above, then the workgroup of a
// row that gets done last adds the row's partial sums in the order of stage 2 - the same value,
// bit for bit, without the second launch and the gap before it.  The partial sums are handed
// over through device-scope stores, each workgroup waits for its own before it draws its ticket,
// and the last one reads them with device-scope loads (no device-wide fence).
// The tickets live in a device array of the library, zero when the library is loaded and left
// zero by every launch; concurrent launches take different slots of it (handed out in turn).
constexpr int SUM_TICKET_SLOTS = 256;
constexpr int SUM_TICKET_ROWS = 64;
__device__ unsigned int sum_tickets[SUM_TICKET_SLOTS][SUM_TICKET_ROWS];

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sum_rows_fused(const T* __restrict__ in, double* __restrict__ partial,
                                                      T* __restrict__ out, int64_t cols, int square, int slot) {
    const int64_t row = blockIdx.y;
    const T* __restrict__ p = in + (size_t)row * cols;
    double acc = 0.0;
    if constexpr (VEC) {
        constexpr int W = 16 / sizeof(T);
        using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
        const V* __restrict__ pv = reinterpret_cast<const V*>(p);
        const int64_t groups = cols / W;
        const int64_t stride = (int64_t)gridDim.x * 256;
        int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
        auto add = [&](const V& v) {
            const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                const double x = (double)e[j];
                acc += square ? x * x : x;
            }
        };
        for (; g + stride < groups; g += 2 * stride) {
            const V a = pv[g];
            const V b = pv[g + stride];
            add(a);
            add(b);
        }
        if (g < groups) add(pv[g]);
    } else {
        const int64_t stride = (int64_t)gridDim.x * 256;
        for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += stride) {
            const double v = (double)p[c];
            acc += square ? v * v : v;
        }
    }
    __shared__ double scratch[4];
    __shared__ unsigned int is_last;
    const int n_partials = (int)gridDim.x;
    const double tot = kmx_block_sum<double>(acc, scratch);
    if (threadIdx.x == 0) {
        __hip_atomic_store(&partial[(size_t)row * n_partials + blockIdx.x], tot, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        unsigned int* ticket = &sum_tickets[slot][row];
        const unsigned int arrived = atomicAdd(ticket, 1u);
        is_last = arrived == (unsigned int)n_partials - 1u ? 1u : 0u;
        if (is_last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (is_last == 0u) return;
    double acc2 = 0.0;
    for (int j = threadIdx.x; j < n_partials; j += 256)
        acc2 += __hip_atomic_load(&partial[(size_t)row * n_partials + j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const double tot2 = kmx_block_sum<double>(acc2, scratch);
    if (threadIdx.x == 0) out[row] = (T)tot2;
}

template <typename T>
__global__ __launch_bounds__(256) void sum_cols_stage1(const T* __restrict__ in,
                                                       double* __restrict__ partial, int64_t rows,
                                                       int64_t cols, int64_t rows_per_chunk) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk;
    int64_t r1 = r0 + rows_per_chunk;
    if (r1 > rows) r1 = rows;
    double acc = 0.0;
    for (int64_t r = r0; r < r1; ++r) acc += (double)in[(size_t)r * cols + c];
    partial[(size_t)blockIdx.y * cols + c] = acc;
}

template <typename T>
__global__ __launch_bounds__(256) void sum_cols_stage2(const double* __restrict__ partial,
                                                       T* __restrict__ out, int64_t cols,
                                                       int n_chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    double acc = 0.0;
    for (int j = 0; j < n_chunks; ++j) acc += partial[(size_t)j * cols + c];
    out[c] = (T)acc;
}

// Single workgroup: n is small wherever the engine needs an argmin (n_local_trials values),
// larger inputs are strided over.
template <typename T>
__global__ __launch_bounds__(1024) void argmin_kernel(const T* __restrict__ values,
                                                      int32_t* __restrict__ out, int64_t n) {
    T best = kmx_inf<T>();
    int64_t arg = INT64_MAX;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const T v = values[i];
        kmx_argmin_combine(best, arg, v, i);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const T ov = __shfl_xor(best, off, 64);
        const int64_t oi = __shfl_xor(arg, off, 64);
        kmx_argmin_combine(best, arg, ov, oi);
    }
    __shared__ T sv[16];
    __shared__ int64_t si[16];
    if ((threadIdx.x & 63) == 0) {
        sv[threadIdx.x >> 6] = best;
        si[threadIdx.x >> 6] = arg;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) kmx_argmin_combine(best, arg, sv[w], si[w]);
        // every value NaN or +inf beyond the first: fall back to the first index
        out[0] = (int32_t)(arg == INT64_MAX ? 0 : arg);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void half_sq_norms_kernel(const T* __restrict__ a_t,
                                                            T* __restrict__ out, int rows,
                                                            int cols) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    T acc = T(0);
    for (int r = 0; r < rows; ++r) {
        const T v = a_t[(size_t)r * cols + c];
        acc += v * v;
    }
    out[c] = acc / T(2);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void broadcast_rows_kernel(T* __restrict__ a,
                                                             const T* __restrict__ v, int64_t rows,
                                                             int64_t cols, int op) {
    const int64_t row = blockIdx.y;
    const T rv = op == 0 ? -v[row] : v[row];
    T* __restrict__ p = a + (size_t)row * cols;
    const int64_t stride = (int64_t)gridDim.x * 256;
    if constexpr (VEC) {
        constexpr int W = 16 / sizeof(T);
        using V = typename std::conditional<sizeof(T) == 4, float4, double2>::type;
        V* __restrict__ pv = reinterpret_cast<V*>(p);
        const int64_t groups = cols / W;
        for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += stride) {
            V x = pv[g];
            T* e = reinterpret_cast<T*>(&x);
#pragma unroll
            for (int j = 0; j < W; ++j) e[j] = e[j] + rv;
            pv[g] = x;
        }
    } else {
        for (int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x; c < cols; c += stride) p[c] = p[c] + rv;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void broadcast_div_cols_kernel(T* __restrict__ a,
                                                                 const T* __restrict__ v,
                                                                 int64_t rows, int64_t cols) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    const T dv = v[c];
    for (int64_t r = 0; r < rows; ++r) a[(size_t)r * cols + c] = a[(size_t)r * cols + c] / dv;
}

template <typename T>
__global__ __launch_bounds__(256) void divide_by_kernel(T* __restrict__ data, int64_t n, T divisor) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        data[i] = data[i] / divisor;
}

__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned char* __restrict__ data,
                                                        int64_t n_bytes) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t n_words = n_bytes / 4;
    uint32_t* w = reinterpret_cast<uint32_t*>(data);
    const bool aligned = (reinterpret_cast<uintptr_t>(data) & 3) == 0;
    if (aligned) {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_words; i += stride) w[i] = 0u;
        for (int64_t i = n_words * 4 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_bytes; i += stride)
            data[i] = 0;
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_bytes; i += stride) data[i] = 0;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void centroid_shifts_kernel(const T* __restrict__ a_t,
                                                              const T* __restrict__ b_t,
                                                              T* __restrict__ out, int d, int k) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= k) return;
    T acc = T(0);
    for (int f = 0; f < d; ++f) {
        const T diff = a_t[(size_t)f * k + c] - b_t[(size_t)f * k + c];
        acc += diff * diff;
    }
    out[c] = acc;
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* __restrict__ p, int64_t n,
                                                       int32_t value, int32_t* extra,
                                                       int32_t extra_value) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) p[i] = value;
    if (extra && blockIdx.x == 0 && threadIdx.x == 0) extra[0] = extra_value;
}

// mapping[l1[i]] = l2[i]; concurrent writers of one slot race, any winner serves: if the two
// labelings agree up to a permutation every writer of a slot stores the same value.
__global__ __launch_bounds__(256) void build_mapping_kernel(const uint32_t* __restrict__ l1,
                                                            const uint32_t* __restrict__ l2,
                                                            int32_t* __restrict__ mapping,
                                                            int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        mapping[l1[i]] = (int32_t)l2[i];
}

__global__ __launch_bounds__(256) void check_mapping_kernel(const uint32_t* __restrict__ l1,
                                                            const uint32_t* __restrict__ l2,
                                                            const int32_t* __restrict__ mapping,
                                                            int32_t* __restrict__ result,
                                                            int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    bool bad = false;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
        bad |= mapping[l1[i]] != (int32_t)l2[i];
    if (__any(bad) && (threadIdx.x & 63) == 0) result[0] = 0;
}

__global__ __launch_bounds__(256) void count_distinct_kernel(const uint32_t* __restrict__ labels,
                                                             int32_t* __restrict__ seen,
                                                             int32_t* __restrict__ result,
                                                             int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const uint32_t l = labels[i];
        if (__builtin_nontemporal_load(seen + l) > 0) continue;
        if (atomicAdd(seen + l, 1) == 0) atomicAdd(result, 1);
    }
}

int grid_for(int64_t n) {
    int64_t blocks = kmx_cdiv(n, 256);
    const int64_t cap = (int64_t)kmx_num_cus() * 8;
    if (blocks > cap) blocks = cap;
    return (int)(blocks < 1 ? 1 : blocks);
}

int sum_blocks_per_row(int64_t cols) {
    int64_t b = kmx_cdiv(cols, 256 * 8);
    if (b > SUM_MAX_BLOCKS_PER_ROW) b = SUM_MAX_BLOCKS_PER_ROW;
    return (int)(b < 1 ? 1 : b);
}


// dst (cols x rows) = transpose of src (rows x cols), 64 x 64 tiles through LDS (rows padded
// by one word: the transposed reads fall on distinct banks); both sides move whole segments.
// One workgroup per tile, tiles numbered along the columns first.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ src, T* __restrict__ dst,
                                                        int64_t rows, int64_t cols, int64_t tiles_c) {
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t r0 = ((int64_t)blockIdx.x / tiles_c) * 64, c0 = ((int64_t)blockIdx.x % tiles_c) * 64;
    const int nr = rows - r0 < 64 ? (int)(rows - r0) : 64, nc = cols - c0 < 64 ? (int)(cols - c0) : 64;
    if (cols <= 64) {
        // narrow source: the tile's rows are one contiguous run of nr * cols elements
        const T* __restrict__ run = src + (size_t)r0 * cols;
        for (int e = threadIdx.x; e < nr * (int)cols; e += 256) tile[e / (int)cols][e % (int)cols] = run[e];
    } else {
#pragma unroll 4
        for (int i = ty; i < 64; i += 4)
            if (i < nr && tx < nc) tile[i][tx] = src[(size_t)(r0 + i) * cols + c0 + tx];
    }
    __syncthreads();
    if (rows <= 64) {
        // narrow result: the tile's columns are one contiguous run of nc * rows elements
        T* __restrict__ run = dst + (size_t)c0 * rows;
        for (int e = threadIdx.x; e < nc * (int)rows; e += 256) run[e] = tile[e % (int)rows][e / (int)rows];
    } else {
#pragma unroll 4
        for (int i = ty; i < 64; i += 4)
            if (i < nc && tx < nr) dst[(size_t)(c0 + i) * rows + r0 + tx] = tile[tx][i];
    }
}

}  // namespace

extern "C" {

size_t kmx_sum_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    const size_t a = (size_t)rows * SUM_MAX_BLOCKS_PER_ROW * sizeof(double);
    const size_t b = (size_t)cols * SUM_COL_CHUNKS * sizeof(double);
    return kmx_align256(a > b ? a : b);
}

int32_t kmx_sum_rows(const void* in, void* out, int64_t rows, int64_t cols, int32_t square,
                     void* workspace, size_t workspace_bytes, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(in);
    KMX_REQUIRE_PTR(out);
    KMX_REQUIRE_PTR(workspace);
    if (rows <= 0 || cols <= 0 || rows > 65535) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    const int b = sum_blocks_per_row(cols);
    if (workspace_bytes < (size_t)rows * b * sizeof(double)) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    double* partial = (double*)workspace;
    const size_t es = kmx_dtype_size(dtype);
    const bool vec = (((uintptr_t)in) % 16 == 0) && ((cols * es) % 16 == 0);
    // Few workgroups (one round of them on the chip): one launch, the last workgroup of a row
    // finishes it (same sums, same order).  The hand-over costs every workgroup two round trips
    // to memory at its end, which a launch of many short workgroups pays for more dearly than
    // for the second launch: 14 rows of 5e6 values took 69 us that way against 45 us.
    static std::atomic<unsigned int> next_slot{0};
    const bool fused = rows <= SUM_TICKET_ROWS && rows * (int64_t)b <= 2 * (int64_t)kmx_num_cus();
    const int slot = fused ? (int)(next_slot.fetch_add(1u) % (unsigned int)SUM_TICKET_SLOTS) : 0;
#define KMX_SUM_ROWS(T, VEC)                                                                       \
    do {                                                                                           \
        if (fused) {                                                                               \
            hipLaunchKernelGGL((sum_rows_fused<T, VEC>), dim3(b, (unsigned)rows), dim3(256), 0, stream, \
                               (const T*)in, partial, (T*)out, cols, square, slot);                \
        } else {                                                                                   \
            hipLaunchKernelGGL((sum_rows_stage1<T, VEC>), dim3(b, (unsigned)rows), dim3(256), 0, stream, \
                               (const T*)in, partial, cols, square);                               \
            hipLaunchKernelGGL((sum_rows_stage2<T>), dim3((unsigned)rows), dim3(256), 0, stream,    \
                               partial, (T*)out, b);                                               \
        }                                                                                          \
    } while (0)
    if (dtype == KMX_F32) {
        if (vec) KMX_SUM_ROWS(float, true); else KMX_SUM_ROWS(float, false);
    } else {
        if (vec) KMX_SUM_ROWS(double, true); else KMX_SUM_ROWS(double, false);
    }
#undef KMX_SUM_ROWS
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

// ---- kmx_sum_rows without any allocation: the per-workgroup partial sums live in a
// file-scope device array instead of a caller-provided workspace.
}  // extern "C"

namespace {
constexpr int SUM_STATIC_MAX_ROWS = 64;
__device__ __align__(256) double sum_static_scratch[SUM_STATIC_MAX_ROWS * SUM_MAX_BLOCKS_PER_ROW];  // 128 KiB

// Device address of sum_static_scratch on the current device (every GPU holds its own copy of
// the array at its own address; the array's name is only a host-side handle and must never be
// handed to a kernel).  Looked up once per device; no allocation.
constexpr int SUM_STATIC_MAX_DEVICES = 64;
int32_t sum_static_scratch_ptr(double** out) {
    static double* ptrs[SUM_STATIC_MAX_DEVICES] = {};
    static std::mutex lock;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int32_t)e;
    if (dev < 0 || dev >= SUM_STATIC_MAX_DEVICES) return KMX_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> guard(lock);
    if (ptrs[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(sum_static_scratch));
        if (e != hipSuccess) return (int32_t)e;
        if (p == nullptr) return KMX_ERR_UNSUPPORTED;
        ptrs[dev] = static_cast<double*>(p);
    }
    *out = ptrs[dev];
    return KMX_OK;
}
}  // namespace

extern "C" {

int32_t kmx_sum_rows_static(const void* in, void* out, int64_t rows, int64_t cols, int32_t square,
                            int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(in);
    KMX_REQUIRE_PTR(out);
    if (rows <= 0 || cols <= 0) return KMX_ERR_BAD_SHAPE;
    if (rows > SUM_STATIC_MAX_ROWS) return KMX_ERR_UNSUPPORTED;  // beyond the static scratch
    KMX_REQUIRE_DTYPE(dtype);
    double* partial = nullptr;
    const int32_t rc = sum_static_scratch_ptr(&partial);
    if (rc != KMX_OK) return rc;
    // stage 1 writes every slot stage 2 reads (rows * b of them), so nothing has to start at
    // zero and the previous call's contents do not matter
    return kmx_sum_rows(in, out, rows, cols, square, partial,
                        sizeof(double) * SUM_STATIC_MAX_ROWS * SUM_MAX_BLOCKS_PER_ROW, dtype, stream_);
}

int32_t kmx_sum_cols(const void* in, void* out, int64_t rows, int64_t cols, void* workspace,
                     size_t workspace_bytes, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(in);
    KMX_REQUIRE_PTR(out);
    KMX_REQUIRE_PTR(workspace);
    if (rows <= 0 || cols <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    int64_t chunks = kmx_cdiv(rows, 64);
    if (chunks > SUM_COL_CHUNKS) chunks = SUM_COL_CHUNKS;
    const int64_t rows_per_chunk = kmx_cdiv(rows, chunks);
    chunks = kmx_cdiv(rows, rows_per_chunk);
    if (workspace_bytes < (size_t)chunks * cols * sizeof(double)) return KMX_ERR_WORKSPACE;
    hipStream_t stream = (hipStream_t)stream_;
    double* partial = (double*)workspace;
    const unsigned gx = (unsigned)kmx_cdiv(cols, 256);
    if (dtype == KMX_F32) {
        hipLaunchKernelGGL((sum_cols_stage1<float>), dim3(gx, (unsigned)chunks), dim3(256), 0,
                           stream, (const float*)in, partial, rows, cols, rows_per_chunk);
        hipLaunchKernelGGL((sum_cols_stage2<float>), dim3(gx), dim3(256), 0, stream, partial,
                           (float*)out, cols, (int)chunks);
    } else {
        hipLaunchKernelGGL((sum_cols_stage1<double>), dim3(gx, (unsigned)chunks), dim3(256), 0,
                           stream, (const double*)in, partial, rows, cols, rows_per_chunk);
        hipLaunchKernelGGL((sum_cols_stage2<double>), dim3(gx), dim3(256), 0, stream, partial,
                           (double*)out, cols, (int)chunks);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_argmin(const void* values, int32_t* out, int64_t n, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(values);
    KMX_REQUIRE_PTR(out);
    if (n <= 0 || n > INT32_MAX) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((argmin_kernel<float>), dim3(1), dim3(1024), 0, stream,
                           (const float*)values, out, n);
    else
        hipLaunchKernelGGL((argmin_kernel<double>), dim3(1), dim3(1024), 0, stream,
                           (const double*)values, out, n);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_half_sq_norms(const void* a_t, void* out, int32_t rows, int32_t cols, int32_t dtype,
                          void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(a_t);
    KMX_REQUIRE_PTR(out);
    if (rows <= 0 || cols <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const unsigned grid = (unsigned)kmx_cdiv(cols, 256);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((half_sq_norms_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (const float*)a_t, (float*)out, rows, cols);
    else
        hipLaunchKernelGGL((half_sq_norms_kernel<double>), dim3(grid), dim3(256), 0, stream,
                           (const double*)a_t, (double*)out, rows, cols);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_transpose(const void* src, void* dst, int64_t rows, int64_t cols, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(src);
    KMX_REQUIRE_PTR(dst);
    if (rows <= 0 || cols <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (src == dst) return KMX_ERR_BAD_ARGUMENT;
    const int64_t tiles_c = kmx_cdiv(cols, 64), tiles = tiles_c * kmx_cdiv(rows, 64);
    if (tiles > INT32_MAX) return KMX_ERR_BAD_SHAPE;
    hipStream_t stream = (hipStream_t)stream_;
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((transpose_kernel<float>), dim3((unsigned)tiles), dim3(256), 0, stream,
                           (const float*)src, (float*)dst, rows, cols, tiles_c);
    else
        hipLaunchKernelGGL((transpose_kernel<double>), dim3((unsigned)tiles), dim3(256), 0, stream,
                           (const double*)src, (double*)dst, rows, cols, tiles_c);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_broadcast_rows(void* a, const void* v, int64_t rows, int64_t cols, int32_t op,
                           int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(a);
    KMX_REQUIRE_PTR(v);
    if (rows <= 0 || cols <= 0 || rows > 65535) return KMX_ERR_BAD_SHAPE;
    if (op != 0 && op != 1) return KMX_ERR_BAD_ARGUMENT;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    int64_t gx = kmx_cdiv(cols, 256 * 4);
    if (gx > 2048) gx = 2048;
    const size_t es = kmx_dtype_size(dtype);
    const bool vec = (((uintptr_t)a) % 16 == 0) && ((cols * es) % 16 == 0);
#define KMX_BCAST(T, VEC)                                                                       \
    hipLaunchKernelGGL((broadcast_rows_kernel<T, VEC>), dim3((unsigned)gx, (unsigned)rows),      \
                       dim3(256), 0, stream, (T*)a, (const T*)v, rows, cols, op)
    if (dtype == KMX_F32) {
        if (vec) KMX_BCAST(float, true); else KMX_BCAST(float, false);
    } else {
        if (vec) KMX_BCAST(double, true); else KMX_BCAST(double, false);
    }
#undef KMX_BCAST
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_broadcast_div_cols(void* a, const void* v, int64_t rows, int64_t cols, int32_t dtype,
                               void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(a);
    KMX_REQUIRE_PTR(v);
    if (rows <= 0 || cols <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const unsigned grid = (unsigned)kmx_cdiv(cols, 256);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((broadcast_div_cols_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (float*)a, (const float*)v, rows, cols);
    else
        hipLaunchKernelGGL((broadcast_div_cols_kernel<double>), dim3(grid), dim3(256), 0, stream,
                           (double*)a, (const double*)v, rows, cols);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_divide_by(void* data, int64_t n_items, double divisor, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(data);
    if (n_items <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const int grid = grid_for(n_items);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((divide_by_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (float*)data, n_items, (float)divisor);
    else
        hipLaunchKernelGGL((divide_by_kernel<double>), dim3(grid), dim3(256), 0, stream,
                           (double*)data, n_items, divisor);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_fill_zero(void* data, int64_t n_bytes, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(data);
    if (n_bytes < 0) return KMX_ERR_BAD_SHAPE;
    if (n_bytes == 0) return KMX_OK;
    hipStream_t stream = (hipStream_t)stream_;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(n_bytes / 4 + 1)), dim3(256), 0, stream,
                       (unsigned char*)data, n_bytes);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_centroid_shifts(const void* a_t, const void* b_t, void* out, int32_t d, int32_t k,
                            int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(a_t);
    KMX_REQUIRE_PTR(b_t);
    KMX_REQUIRE_PTR(out);
    if (d <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const unsigned grid = (unsigned)kmx_cdiv(k, 256);
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((centroid_shifts_kernel<float>), dim3(grid), dim3(256), 0, stream,
                           (const float*)a_t, (const float*)b_t, (float*)out, d, k);
    else
        hipLaunchKernelGGL((centroid_shifts_kernel<double>), dim3(grid), dim3(256), 0, stream,
                           (const double*)a_t, (const double*)b_t, (double*)out, d, k);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_is_same_clustering(const uint32_t* labels1, const uint32_t* labels2, int32_t* mapping,
                               int32_t* result, int64_t n, int32_t k, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(labels1);
    KMX_REQUIRE_PTR(labels2);
    KMX_REQUIRE_PTR(mapping);
    KMX_REQUIRE_PTR(result);
    if (n <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    hipStream_t stream = (hipStream_t)stream_;
    const int grid = grid_for(n);
    hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, stream, mapping, (int64_t)k, -1,
                       result, 1);
    hipLaunchKernelGGL(build_mapping_kernel, dim3(grid), dim3(256), 0, stream, labels1, labels2,
                       mapping, n);
    hipLaunchKernelGGL(check_mapping_kernel, dim3(grid), dim3(256), 0, stream, labels1, labels2,
                       mapping, result, n);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_count_distinct_clusters(const uint32_t* labels, int32_t* seen, int32_t* result,
                                    int64_t n, int32_t k, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(labels);
    KMX_REQUIRE_PTR(seen);
    KMX_REQUIRE_PTR(result);
    if (n <= 0 || k <= 0) return KMX_ERR_BAD_SHAPE;
    hipStream_t stream = (hipStream_t)stream_;
    hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, stream, seen, (int64_t)k, 0, result,
                       0);
    hipLaunchKernelGGL(count_distinct_kernel, dim3(grid_for(n)), dim3(256), 0, stream, labels, seen,
                       result, n);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

}  // extern "C"
