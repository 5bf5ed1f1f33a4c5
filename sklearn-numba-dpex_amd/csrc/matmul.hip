// out (m, q) = X (m, p) @ Y_t (q, p)^T for gfx950.  Not on the KMeans call path (the reference
// only calls make_matmul_2d_kernel, common/matmul.py:13-567, from its own test); kept for
// parity of the shared-kernel surface.
//
//   * fp32: matrix cores (v_mfma_f32_32x32x2_f32).  A workgroup of four waves owns a 128 x 128
//     output tile, a wave a 64 x 64 quarter of it (2 x 2 MFMA tiles, 64 accumulator registers).
//     Both operands have K innermost in memory; a thread reads four consecutive K values of
//     one row with a 128-bit load and stores them K-major into LDS ([kk][row], double
//     buffered, 16 K values per stage), so that the fragment reads of a half-wave are 32
//     consecutive words.  The next stage's global loads are in flight during the MFMAs.
//   * fp64: matrix cores (v_mfma_f64_16x16x4_f64), the same 128 x 128 workgroup tile and
//     64 x 64 wave quarter (4 x 4 MFMA tiles, 64 accumulator doubles per lane), K staged 16 at
//     a time through K-major LDS tiles; a thread reads two consecutive K values per 128-bit load.
//   * tiny shapes, and a `multiply` other than the product (x - y or x + y summed over K, which
//     is no matrix product): LDS-tiled vector-ALU kernel, 64 x 64 output tile per workgroup of
//     256 threads, 4 x 4 register block per thread, K staged 16 at a time.
//   * every kernel applies the output function (identity, square, division by a constant) to
//     the finished sum in its epilogue.
#include "kmx_common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef double v4d __attribute__((ext_vector_type(4)));

// out_fused_elementwise_fn of the reference (common/matmul.py:55-62) for its predefined
// functions (common/_utils.py:17-33): applied once to every finished sum.
template <typename T>
__device__ __forceinline__ T mm_finish(T v, int out_op, T out_param) {
    if (out_op == KMX_MATMUL_OUT_SQUARE) return v * v;
    if (out_op == KMX_MATMUL_OUT_DIVIDE_BY) return v / out_param;
    return v;
}

// multiply_fn of the reference (common/matmul.py:64-66): the scalar combined over K.
template <int MUL, typename T>
__device__ __forceinline__ T mm_combine(T x, T y, T acc) {
    if constexpr (MUL == KMX_MATMUL_MINUS) return acc + (x - y);
    else if constexpr (MUL == KMX_MATMUL_PLUS) return acc + (x + y);
    else return fma(x, y, acc);
}

constexpr int MM = 128, MN = 128, MK = 16;  // MFMA kernel: workgroup tile and K stage

// Stage loads: the 128 x 16 tile of an operand is 512 groups of four K values; thread t takes
// groups t and t + 256: row (g / 4), K offset 4 (g % 4).
__device__ __forceinline__ void mm_stage_load(float4 (&r)[2], const float* __restrict__ base, int rows,
                                              int row0, int p, int k0, bool vec_ok) {
#pragma unroll
    for (int l = 0; l < 2; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int row = row0 + (g >> 2), kk = k0 + 4 * (g & 3);
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row < rows) {
            const float* __restrict__ src = base + (size_t)row * p + kk;
            if (vec_ok && kk + 4 <= p) {
                v = *reinterpret_cast<const float4*>(src);
            } else {
                if (kk + 0 < p) v.x = src[0];
                if (kk + 1 < p) v.y = src[1];
                if (kk + 2 < p) v.z = src[2];
                if (kk + 3 < p) v.w = src[3];
            }
        }
        r[l] = v;
    }
}

__device__ __forceinline__ void mm_stage_store(float (*tile)[MM], const float4 (&r)[2]) {
#pragma unroll
    for (int l = 0; l < 2; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int row = g >> 2, kk = 4 * (g & 3);
        tile[kk + 0][row] = r[l].x;
        tile[kk + 1][row] = r[l].y;
        tile[kk + 2][row] = r[l].z;
        tile[kk + 3][row] = r[l].w;
    }
}

__global__ __launch_bounds__(256) void matmul_mfma_f32_kernel(const float* __restrict__ X,
                                                              const float* __restrict__ Y_t,
                                                              float* __restrict__ out, int m, int p,
                                                              int q, int vec_ok, int out_op, float out_param) {
    __shared__ float xs[2][MK][MM];
    __shared__ float ys[2][MK][MN];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = lane >> 5, j = lane & 31;
    const int row0 = blockIdx.y * MM, col0 = blockIdx.x * MN;
    const int wr = 64 * (wave >> 1), wc = 64 * (wave & 1);  // the wave's quarter of the tile

    v16f acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    float4 rx[2], ry[2];
    mm_stage_load(rx, X, m, row0, p, 0, vec_ok != 0);
    mm_stage_load(ry, Y_t, q, col0, p, 0, vec_ok != 0);
    mm_stage_store(xs[0], rx);
    mm_stage_store(ys[0], ry);
    __syncthreads();

    const int n_stages = (p + MK - 1) / MK;
    for (int st = 0; st < n_stages; ++st) {
        const int cur = st & 1;
        if (st + 1 < n_stages) {
            mm_stage_load(rx, X, m, row0, p, (st + 1) * MK, vec_ok != 0);
            mm_stage_load(ry, Y_t, q, col0, p, (st + 1) * MK, vec_ok != 0);
        }
#pragma unroll
        for (int s = 0; s < MK / 2; ++s) {
            // MFMA operands: lane (i, h) supplies K index 2 s + h of row / column i
            float af[2], bf[2];
#pragma unroll
            for (int a = 0; a < 2; ++a) af[a] = xs[cur][2 * s + h][wr + 32 * a + j];
#pragma unroll
            for (int b = 0; b < 2; ++b) bf[b] = ys[cur][2 * s + h][wc + 32 * b + j];
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[a], bf[b], acc[a][b], 0, 0, 0);
        }
        if (st + 1 < n_stages) {
            mm_stage_store(xs[cur ^ 1], rx);
            mm_stage_store(ys[cur ^ 1], ry);
        }
        __syncthreads();
    }

    // accumulator register r of lane (j, h): row 8 (r / 4) + 4 h + r % 4, column j of the tile
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const int gc = col0 + wc + 32 * b + j;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int gr = row0 + wr + 32 * a + 8 * (r >> 2) + 4 * h + (r & 3);
                if (gr < m && gc < q) out[(size_t)gr * q + gc] = mm_finish(acc[a][b][r], out_op, out_param);
            }
        }
}

// fp64 stage loads: the 128 x 16 tile of an operand is 1024 pairs of K values; thread t takes
// pairs t + 256 l (l < 4): row (g / 8), K offset 2 (g % 8).
__device__ __forceinline__ void mm_stage_load_f64(double2 (&r)[4], const double* __restrict__ base, int rows,
                                                  int row0, int p, int k0, bool vec_ok) {
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int row = row0 + (g >> 3), kk = k0 + 2 * (g & 7);
        double2 v = make_double2(0.0, 0.0);
        if (row < rows) {
            const double* __restrict__ src = base + (size_t)row * p + kk;
            if (vec_ok && kk + 2 <= p) {
                v = *reinterpret_cast<const double2*>(src);
            } else {
                if (kk + 0 < p) v.x = src[0];
                if (kk + 1 < p) v.y = src[1];
            }
        }
        r[l] = v;
    }
}

__device__ __forceinline__ void mm_stage_store_f64(double (*tile)[MM], const double2 (&r)[4]) {
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        const int g = threadIdx.x + 256 * l;
        const int row = g >> 3, kk = 2 * (g & 7);
        tile[kk + 0][row] = r[l].x;
        tile[kk + 1][row] = r[l].y;
    }
}

// v_mfma_f64_16x16x4_f64: lane l = (g, j) = (l / 16, l % 16) supplies A[row j][K g] and
// B[K g][column j], and holds D[rows g + 4 r, r = 0..3][column j].
__global__ __launch_bounds__(256) void matmul_mfma_f64_kernel(const double* __restrict__ X,
                                                              const double* __restrict__ Y_t,
                                                              double* __restrict__ out, int m, int p, int q,
                                                              int vec_ok, int out_op, double out_param) {
    __shared__ double xs[MK][MM];
    __shared__ double ys[MK][MN];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 4, j = lane & 15;
    const int row0 = blockIdx.y * MM, col0 = blockIdx.x * MN;
    const int wr = 64 * (wave >> 1), wc = 64 * (wave & 1);  // the wave's quarter of the tile

    v4d acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[a][b][r] = 0.0;

    double2 rx[4], ry[4];
    mm_stage_load_f64(rx, X, m, row0, p, 0, vec_ok != 0);
    mm_stage_load_f64(ry, Y_t, q, col0, p, 0, vec_ok != 0);

    const int n_stages = (p + MK - 1) / MK;
    for (int st = 0; st < n_stages; ++st) {
        mm_stage_store_f64(xs, rx);
        mm_stage_store_f64(ys, ry);
        __syncthreads();
        if (st + 1 < n_stages) {  // in flight during the MFMAs
            mm_stage_load_f64(rx, X, m, row0, p, (st + 1) * MK, vec_ok != 0);
            mm_stage_load_f64(ry, Y_t, q, col0, p, (st + 1) * MK, vec_ok != 0);
        }
#pragma unroll
        for (int s = 0; s < MK / 4; ++s) {
            double af[4], bf[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) af[a] = xs[4 * s + g][wr + 16 * a + j];
#pragma unroll
            for (int b = 0; b < 4; ++b) bf[b] = ys[4 * s + g][wc + 16 * b + j];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[a], bf[b], acc[a][b], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int gc = col0 + wc + 16 * b + j;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int gr = row0 + wr + 16 * a + g + 4 * r;
                if (gr < m && gc < q) out[(size_t)gr * q + gc] = mm_finish(acc[a][b][r], out_op, out_param);
            }
        }
}

constexpr int TM = 64, TN = 64, TK = 16;

template <typename T, int MUL>
__global__ __launch_bounds__(256) void matmul_kernel(const T* __restrict__ X,
                                                     const T* __restrict__ Y_t,
                                                     T* __restrict__ out, int m, int p, int q, int out_op,
                                                     T out_param) {
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
        // K values past p are zero in both tiles: they add nothing for any of the three combinations
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
                for (int j = 0; j < 4; ++j) acc[i][j] = mm_combine<MUL>(a[i], b[j], acc[i][j]);
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
            if (gc < q) out[(size_t)gr * q + gc] = mm_finish(acc[i][j], out_op, out_param);
        }
    }
}

template <typename T, int MUL>
void launch_valu(const void* X, const void* Y_t, void* out, int m, int p, int q, int out_op, double out_param,
                 hipStream_t stream) {
    const dim3 grid((unsigned)kmx_cdiv(q, TN), (unsigned)kmx_cdiv(m, TM));
    hipLaunchKernelGGL((matmul_kernel<T, MUL>), grid, dim3(256), 0, stream, (const T*)X, (const T*)Y_t, (T*)out, m,
                       p, q, out_op, (T)out_param);
}

}  // namespace

extern "C" {

int32_t kmx_matmul_fused(const void* X, const void* Y_t, void* out, int32_t m, int32_t p, int32_t q,
                         int32_t multiply_op, int32_t out_op, double out_param, int32_t dtype, void* stream_) {
    KMX_ENTRY();
    KMX_REQUIRE_PTR(X);
    KMX_REQUIRE_PTR(Y_t);
    KMX_REQUIRE_PTR(out);
    if (m <= 0 || p <= 0 || q <= 0) return KMX_ERR_BAD_SHAPE;
    KMX_REQUIRE_DTYPE(dtype);
    if (multiply_op < KMX_MATMUL_MULTIPLY || multiply_op > KMX_MATMUL_PLUS) return KMX_ERR_BAD_ARGUMENT;
    if (out_op < KMX_MATMUL_OUT_IDENTITY || out_op > KMX_MATMUL_OUT_DIVIDE_BY) return KMX_ERR_BAD_ARGUMENT;
    hipStream_t stream = (hipStream_t)stream_;
    const size_t es = kmx_dtype_size(dtype);
    if (multiply_op == KMX_MATMUL_MULTIPLY && (int64_t)m * q >= 128 * 128) {
        const dim3 mgrid((unsigned)kmx_cdiv(q, MN), (unsigned)kmx_cdiv(m, MM));
        const int vec_ok = ((p * es) % 16 == 0) && ((((uintptr_t)X) & 15) == 0) && ((((uintptr_t)Y_t) & 15) == 0);
        if (dtype == KMX_F32)
            hipLaunchKernelGGL(matmul_mfma_f32_kernel, mgrid, dim3(256), 0, stream, (const float*)X,
                               (const float*)Y_t, (float*)out, m, p, q, vec_ok, out_op, (float)out_param);
        else
            hipLaunchKernelGGL(matmul_mfma_f64_kernel, mgrid, dim3(256), 0, stream, (const double*)X,
                               (const double*)Y_t, (double*)out, m, p, q, vec_ok, out_op, out_param);
        KMX_LAUNCH_CHECK();
        return KMX_OK;
    }
    if (dtype == KMX_F32) {
        if (multiply_op == KMX_MATMUL_MINUS) launch_valu<float, KMX_MATMUL_MINUS>(X, Y_t, out, m, p, q, out_op, out_param, stream);
        else if (multiply_op == KMX_MATMUL_PLUS) launch_valu<float, KMX_MATMUL_PLUS>(X, Y_t, out, m, p, q, out_op, out_param, stream);
        else launch_valu<float, KMX_MATMUL_MULTIPLY>(X, Y_t, out, m, p, q, out_op, out_param, stream);
    } else {
        if (multiply_op == KMX_MATMUL_MINUS) launch_valu<double, KMX_MATMUL_MINUS>(X, Y_t, out, m, p, q, out_op, out_param, stream);
        else if (multiply_op == KMX_MATMUL_PLUS) launch_valu<double, KMX_MATMUL_PLUS>(X, Y_t, out, m, p, q, out_op, out_param, stream);
        else launch_valu<double, KMX_MATMUL_MULTIPLY>(X, Y_t, out, m, p, q, out_op, out_param, stream);
    }
    KMX_LAUNCH_CHECK();
    return KMX_OK;
}

int32_t kmx_matmul(const void* X, const void* Y_t, void* out, int32_t m, int32_t p, int32_t q, int32_t dtype,
                   void* stream) {
    return kmx_matmul_fused(X, Y_t, out, m, p, q, KMX_MATMUL_MULTIPLY, KMX_MATMUL_OUT_IDENTITY, 0.0, dtype, stream);
}

}  // extern "C"
