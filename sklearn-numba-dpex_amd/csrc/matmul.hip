// out (m, q) = X (m, p) @ Y_t (q, p)^T for gfx950: LDS-tiled, 64 x 64 output tile per
// workgroup of 256 threads, 4 x 4 register block per thread, K staged 16 at a time.  LDS
// tiles are stored K-major with a one-element pad so that the 4-wide reads of a register
// block do not collide on banks.  Not on the KMeans call path (the reference only calls it
// from its own test); kept for parity of the shared-kernel surface.
#include "kmx_common.h"

namespace {

constexpr int TM = 64, TN = 64, TK = 16;

template <typename T>
__global__ __launch_bounds__(256) void matmul_kernel(const T* __restrict__ X,
                                                     const T* __restrict__ Y_t,
                                                     T* __restrict__ out, int m, int p, int q) {
    __shared__ T xs[TK][TM + 1];
    __shared__ T ys[TK][TN + 1];
    const int tx = threadIdx.x & 15;   // column group
    const int ty = threadIdx.x >> 4;   // row group
    const int row0 = blockIdx.y * TM;
    const int col0 = blockIdx.x * TN;

    T acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = T(0);

    for (int k0 = 0; k0 < p; k0 += TK) {
        // each thread loads 4 elements of each operand tile (64 rows x 16 k)
#pragma unroll
        for (int l = 0; l < 4; ++l) {
            const int e = threadIdx.x + l * 256;
            const int r = e >> 4, kk = e & 15;
            const int gr = row0 + r, gc = col0 + r, gk = k0 + kk;
            xs[kk][r] = (gr < m && gk < p) ? X[(size_t)gr * p + gk] : T(0);
            ys[kk][r] = (gc < q && gk < p) ? Y_t[(size_t)gc * p + gk] : T(0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            T a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ys[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fma(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gr = row0 + ty * 4 + i;
        if (gr >= m) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gc = col0 + tx * 4 + j;
            if (gc < q) out[(size_t)gr * q + gc] = acc[i][j];
        }
    }
}

}  // namespace

extern "C" int32_t kmx_matmul(const void* X, const void* Y_t, void* out, int32_t m, int32_t p,
                              int32_t q, int32_t dtype, void* stream_) {
    KMX_REQUIRE_PTR(X);
    KMX_REQUIRE_PTR(Y_t);
    KMX_REQUIRE_PTR(out);
    if (m <= 0 || p <= 0 || q <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    hipStream_t stream = (hipStream_t)stream_;
    const dim3 grid((unsigned)kmx_cdiv(q, TN), (unsigned)kmx_cdiv(m, TM));
    if (dtype == KMX_F32)
        hipLaunchKernelGGL((matmul_kernel<float>), grid, dim3(256), 0, stream, (const float*)X,
                           (const float*)Y_t, (float*)out, m, p, q);
    else
        hipLaunchKernelGGL((matmul_kernel<double>), grid, dim3(256), 0, stream, (const double*)X,
                           (const double*)Y_t, (double*)out, m, p, q);
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}
