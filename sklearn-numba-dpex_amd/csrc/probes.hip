// Machine probes: what this GPU reaches on a plain copy, a read-only stream and a stream of
// independent matrix-core instructions.  The benchmark prices the KMeans kernels against these
// measured ceilings next to the datasheet ones.  Nothing of the KMeans path runs through here.
#include "kmx_common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef double v4d __attribute__((ext_vector_type(4)));

// dst[i] = src[i], 16 bytes per lane and step, grid-stride.
__global__ __launch_bounds__(256) void probe_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                          size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += stride) dst[i] = src[i];
}

// Reads src once (four independent 16-byte loads per lane and step) and folds it into one word
// per workgroup, so that the loads cannot be dropped.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, uint32_t* __restrict__ out,
                                                          size_t n_vec) {
    const size_t stride = (size_t)gridDim.x * 256;
    uint32_t acc = 0;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        const uint4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], e = src[i + 3 * stride];
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ e.x ^ e.y ^ e.z ^ e.w;
    }
    for (; i < n_vec; i += stride) {
        const uint4 a = src[i];
        acc ^= a.x ^ a.y ^ a.z ^ a.w;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, 64);
    if ((threadIdx.x & 63) == 0 && acc == 0x9e3779b9u) out[blockIdx.x] = acc;  // practically never
}

// `iters` rounds of four independent accumulation chains per wave, two waves per SIMD.
// KIND 0: v_mfma_f32_32x32x2_f32, 1: v_mfma_f32_32x32x16_f16, 2: v_mfma_f64_16x16x4_f64.
template <int KIND>
__global__ __launch_bounds__(512) void probe_mfma_kernel(float* __restrict__ out, int iters) {
    const float seed = (float)(threadIdx.x & 63) * 0.001f;
    float total = 0.0f;
    if constexpr (KIND == 0) {
        v16f c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        const float a = seed, b = 1.0f - seed;
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, a, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, a, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x2f32(b, b, c3, 0, 0, 0);
        }
        for (int r = 0; r < 16; ++r) total += c0[r] + c1[r] + c2[r] + c3[r];
    } else if constexpr (KIND == 1) {
        v16f c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        v8h a, b;
        for (int i = 0; i < 8; ++i) {
            a[i] = (_Float16)(seed + (float)i);
            b[i] = (_Float16)(1.0f - seed);
        }
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, a, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, a, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(b, b, c3, 0, 0, 0);
        }
        for (int r = 0; r < 16; ++r) total += c0[r] + c1[r] + c2[r] + c3[r];
    } else {
        v4d c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        const double a = seed, b = 1.0 - seed;
        for (int it = 0; it < iters; ++it) {
            c0 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f64_16x16x4f64(b, a, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f64_16x16x4f64(a, a, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f64_16x16x4f64(b, b, c3, 0, 0, 0);
        }
        for (int r = 0; r < 4; ++r) total += (float)(c0[r] + c1[r] + c2[r] + c3[r]);
    }
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = total;
}

// How matrix-core and vector-ALU instructions of one SIMD share its issue slots: every loop
// round issues two independent MFMAs (KIND 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_32x32x2_f32,
// 2: none) and 2 * VALU independent v_max3_f32 on private registers; three waves per SIMD.
template <int KIND, int VALU>
__global__ __launch_bounds__(768) void probe_issue_kernel(float* __restrict__ out, int iters) {
    const float seed = (float)(threadIdx.x & 63) * 0.001f;
    v16f c0 = {0}, c1 = {0};
    v8h ah, bh;
    for (int i = 0; i < 8; ++i) {
        ah[i] = (_Float16)(seed + (float)i);
        bh[i] = (_Float16)(1.0f - seed);
    }
    float r[8];
    for (int i = 0; i < 8; ++i) r[i] = seed + (float)i;
    for (int it = 0; it < iters; ++it) {
        if constexpr (KIND == 0) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(bh, ah, c1, 0, 0, 0);
        } else if constexpr (KIND == 1) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x2f32(seed, 1.0f - seed, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x2f32(1.0f - seed, seed, c1, 0, 0, 0);
        }
#pragma unroll
        for (int q = 0; q < 2 * VALU; ++q)
            asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(r[q & 7]) : "v"(r[(q + 1) & 7]), "v"(r[(q + 3) & 7]));
    }
    float total = 0.0f;
    for (int i = 0; i < 8; ++i) total += r[i];
    for (int i = 0; i < 16; ++i) total += c0[i] + c1[i];
    out[(size_t)blockIdx.x * 768 + threadIdx.x] = total;
}

template <int KIND>
bool launch_issue(int valu, unsigned grid, hipStream_t stream, float* out, int iters) {
    switch (valu) {
        case 0: hipLaunchKernelGGL((probe_issue_kernel<KIND, 0>), dim3(grid), dim3(768), 0, stream, out, iters); return true;
        case 8: hipLaunchKernelGGL((probe_issue_kernel<KIND, 8>), dim3(grid), dim3(768), 0, stream, out, iters); return true;
        case 16: hipLaunchKernelGGL((probe_issue_kernel<KIND, 16>), dim3(grid), dim3(768), 0, stream, out, iters); return true;
        case 32: hipLaunchKernelGGL((probe_issue_kernel<KIND, 32>), dim3(grid), dim3(768), 0, stream, out, iters); return true;
        default: return false;
    }
}

}  // namespace

extern "C" {

int32_t kmx_probe_issue(int32_t kind, int32_t valu_per_mfma, int32_t iters, void* scratch, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(scratch);
    if (iters <= 0) return KMX_ERR_BAD_SHAPE;
    const unsigned grid = (unsigned)kmx_num_cus();
    hipStream_t stream = (hipStream_t)stream_;
    bool ok = false;
    if (kind == 0) ok = launch_issue<0>(valu_per_mfma, grid, stream, (float*)scratch, iters);
    else if (kind == 1) ok = launch_issue<1>(valu_per_mfma, grid, stream, (float*)scratch, iters);
    else if (kind == 2) ok = launch_issue<2>(valu_per_mfma, grid, stream, (float*)scratch, iters);
    if (!ok) return KMX_ERR_BAD_ARGUMENT;
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_probe_copy(const void* src, void* dst, size_t n_bytes, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(src);
    KMX_REQUIRE_PTR(dst);
    if (n_bytes == 0 || n_bytes % 16 != 0 || (((uintptr_t)src | (uintptr_t)dst) & 15) != 0) return KMX_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)(kmx_num_cus() * 8)), dim3(256), 0, (hipStream_t)stream_,
                       (const uint4*)src, (uint4*)dst, n_bytes / 16);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_probe_read(const void* src, size_t n_bytes, void* scratch, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(src);
    KMX_REQUIRE_PTR(scratch);
    if (n_bytes == 0 || n_bytes % 16 != 0 || (((uintptr_t)src) & 15) != 0) return KMX_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)(kmx_num_cus() * 8)), dim3(256), 0, (hipStream_t)stream_,
                       (const uint4*)src, (uint32_t*)scratch, n_bytes / 16);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_probe_mfma(int32_t kind, int32_t iters, void* scratch, double* flops_host, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(scratch);
    KMX_REQUIRE_PTR(flops_host);
    if (iters <= 0) return KMX_ERR_BAD_SHAPE;
    const unsigned grid = (unsigned)kmx_num_cus();
    hipStream_t stream = (hipStream_t)stream_;
    // flops of one instruction: 2 * M * N * K
    double per_inst;
    switch (kind) {
        case 0:
            hipLaunchKernelGGL((probe_mfma_kernel<0>), dim3(grid), dim3(512), 0, stream, (float*)scratch, iters);
            per_inst = 2.0 * 32 * 32 * 2;
            break;
        case 1:
            hipLaunchKernelGGL((probe_mfma_kernel<1>), dim3(grid), dim3(512), 0, stream, (float*)scratch, iters);
            per_inst = 2.0 * 32 * 32 * 16;
            break;
        case 2:
            hipLaunchKernelGGL((probe_mfma_kernel<2>), dim3(grid), dim3(512), 0, stream, (float*)scratch, iters);
            per_inst = 2.0 * 16 * 16 * 4;
            break;
        default: return KMX_ERR_BAD_ARGUMENT;
    }
    KMX_LAUNCH_CHECK();
    *flops_host = per_inst * 4.0 * (double)iters * 8.0 * (double)grid;  // 4 chains, 8 waves per workgroup
    return KMX_OK;
}

}  // extern "C"
