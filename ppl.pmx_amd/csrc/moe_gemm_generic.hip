// Grouped expert GEMM, shape-agnostic fallback (any K, N, dtype incl. fp32).
// Plain LDS-tiled FMA kernel with full bounds checks: used for fp32 tensors and
// for shapes the MFMA kernels do not cover.  fp32 accumulation, one rounding.
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67 and
// torch_function/MoeRowParallelLinear.py:47-53 of OpenPPL/ppl.pmx.
#include "moe_gemm.h"

namespace opmx {
namespace {

constexpr int GB = 64;    // tile is GB x GB outputs
constexpr int GK = 16;    // k step

template <typename T, bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T *__restrict__ X, const int64_t *__restrict__ off,
                                                           const T *__restrict__ W, const T *__restrict__ Bias,
                                                           int E, int64_t R, int64_t K, int64_t N,
                                                           T *__restrict__ Y, const int32_t *__restrict__ rt,
                                                           int64_t xrows)
{
    __shared__ float As[GK][GB + 4];
    __shared__ float Bs[SWIGLU ? 2 : 1][GK][GB + 4];
    const int64_t ncols = SWIGLU ? N / 2 : N;      // output columns
    zero_unowned_rows(Y, R, ncols, off, E);
    const MTile mt = find_mtile(off, E, R, GB, blockIdx.y);
    if (mt.rows == 0) return;
    const int64_t n0 = static_cast<int64_t>(blockIdx.x) * GB;
    const T *We = W + static_cast<int64_t>(mt.e) * N * K;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;

    float acc[SWIGLU ? 2 : 1][4][4];
#pragma unroll
    for (int h = 0; h < (SWIGLU ? 2 : 1); ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[h][i][j] = 0.0f;

    for (int64_t k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int i = 0; i < GB * GK / 256; ++i) {
            const int q = threadIdx.x + 256 * i;
            const int row = q / GK, kk = q % GK;
            const bool kin = k0 + kk < K;
            // the X row of tile row `row`: in place, or through the row index (RowGather)
            const int64_t xr = (rt && row < mt.rows) ? gathered_row(rt, xrows, mt.row0 + row) : mt.row0 + row;
            As[kk][row] = (row < mt.rows && kin) ? to_f32(X[xr * K + k0 + kk]) : 0.0f;
#pragma unroll
            for (int h = 0; h < (SWIGLU ? 2 : 1); ++h) {
                const int64_t n = n0 + row;
                Bs[h][kk][row] = (n < ncols && kin) ? to_f32(We[(n + h * ncols) * K + k0 + kk]) : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            float a[4], b[SWIGLU ? 2 : 1][4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int h = 0; h < (SWIGLU ? 2 : 1); ++h)
#pragma unroll
                for (int j = 0; j < 4; ++j) b[h][j] = Bs[h][kk][tx * 4 + j];
#pragma unroll
            for (int h = 0; h < (SWIGLU ? 2 : 1); ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[h][i][j] += a[i] * b[h][j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = ty * 4 + i;
        if (row >= mt.rows) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n >= ncols) continue;
            float v = acc[0][i][j];
            if (Bias) v += to_f32(Bias[static_cast<int64_t>(mt.e) * N + n]);
            if (SWIGLU) {
                float g = acc[1][i][j];
                if (Bias) g += to_f32(Bias[static_cast<int64_t>(mt.e) * N + ncols + n]);
                v = g * v * sigmoidf_(v);
            }
            Y[(mt.row0 + row) * ncols + n] = from_f32<T>(v);
        }
    }
}

template <typename T>
int generic_impl(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                 int64_t N, int epilogue, void *Y, hipStream_t s, RowGather g)
{
    const int64_t ncols = epilogue == OPMX_EPILOGUE_SWIGLU ? N / 2 : N;
    dim3 grid(static_cast<unsigned>(ceil_div(ncols, GB)), static_cast<unsigned>(max_mtiles(R, E, GB)));
    if (epilogue == OPMX_EPILOGUE_SWIGLU)
        gemm_generic_kernel<T, true><<<grid, 256, 0, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                                          static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), g.index, g.x_rows);
    else
        gemm_generic_kernel<T, false><<<grid, 256, 0, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                                           static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), g.index, g.x_rows);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

int launch_gemm_generic(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                        int64_t K, int64_t N, int dtype, int epilogue, void *Y, hipStream_t s, RowGather g)
{
    switch (dtype) {
        case OPMX_DTYPE_F32: return generic_impl<float>(X, off, W, B, E, R, K, N, epilogue, Y, s, g);
        case OPMX_DTYPE_F16: return generic_impl<f16>(X, off, W, B, E, R, K, N, epilogue, Y, s, g);
        case OPMX_DTYPE_BF16: return generic_impl<bf16>(X, off, W, B, E, R, K, N, epilogue, Y, s, g);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
