// SwiGLU and gated SiLU for gfx950 (elementwise, HBM bound, 16 bytes per lane).
// Semantics: torch_function/SwiGLU.py:15-16 and torch_function/SiLU.py:18-21.
#include "common.h"

namespace opmx {
namespace {

// sigmoid for an output of type T: the accurate routine (expf and an IEEE division, some 30
// instructions) for fp32 tensors; hardware exp2 and reciprocal (1 ulp each in fp32) where the
// result is rounded to 16 bits anyway.  With the accurate one the 16-bit kernels are bound by the
// vector ALUs, not by memory (-8 % on SwiGLU over [16384, 2 x 14336] fp16).
template <typename T> __device__ __forceinline__ float sigmoid_for(float x)
{
    if constexpr (sizeof(T) == 2) return sigmoid_fast_(x);
    else return sigmoidf_(x);
}

// Y[r,i] = (g * x) * sigmoid(beta*x), x = X[r,i], g = X[r,D+i].  A block takes one row of one
// 256-chunk column strip (16 bytes per lane) and lives for that long only, so the grid (x over
// the strips fastest, then the rows) sweeps the tensors front to back the way a plain elementwise
// kernel does.  Measured on [16384, 2 x 14336] fp16 (1.4 GB of traffic): 224 us = 6.3 TB/s, against
// 236 us for a plain product with the same traffic; long-lived blocks that walk the rows with a
// stride of a few hundred ran at 4.9 TB/s, four consecutive rows per block at 5.5.
template <typename T>
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const T *__restrict__ X, int64_t R, int64_t D, float beta,
                                                         T *__restrict__ Y)
{
    constexpr int n = Vec16<T>::n;
    const int64_t c = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * n;
    if (c >= D) return;
    for (int64_t r = blockIdx.y; r < R; r += gridDim.y) {
        const Vec16<T> x = load16_once(X + r * 2 * D + c), g = load16_once(X + r * 2 * D + D + c);
        Vec16<T> o;
#pragma unroll
        for (int j = 0; j < n; ++j) {
            const float a = to_f32(x.v[j]);
            o.v[j] = from_f32<T>(to_f32(g.v[j]) * a * sigmoid_for<T>(beta * a));
        }
        store16(Y + r * D + c, o);
    }
}

// Rows that are not whole 16-byte chunks, or unaligned tensors: one element per lane.
template <typename T>
__global__ __launch_bounds__(256) void swiglu_scalar_kernel(const T *__restrict__ X, int64_t R, int64_t D, float beta,
                                                            T *__restrict__ Y)
{
    const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (c >= D) return;
    for (int64_t r = blockIdx.y; r < R; r += gridDim.y) {
        const float xf = to_f32(X[r * 2 * D + c]), gf = to_f32(X[r * 2 * D + D + c]);
        Y[r * D + c] = from_f32<T>(gf * xf * sigmoid_for<T>(beta * xf));
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void silu_kernel(const T *__restrict__ X, const T *__restrict__ gate, int64_t cnt,
                                                   T *__restrict__ Y)
{
    constexpr int n = VEC ? Vec16<T>::n : 1;
    const int64_t total = cnt / n;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        if (VEC) {
            Vec16<T> x = load16(X + i * n), g, o;
            if (gate) g = load16(gate + i * n);
#pragma unroll
            for (int j = 0; j < n; ++j) {
                float xf = to_f32(x.v[j]);
                float y = xf * sigmoid_for<T>(xf);
                o.v[j] = from_f32<T>(gate ? to_f32(g.v[j]) * y : y);
            }
            store16(Y + i * n, o);
        } else {
            float xf = to_f32(X[i]);
            float y = xf * sigmoid_for<T>(xf);
            Y[i] = from_f32<T>(gate ? to_f32(gate[i]) * y : y);
        }
    }
}

// One 256-lane block per 256 work items (the kernel strides on only past 2^31 - 1 blocks): short
// blocks in address order stream faster than a few long-lived ones (see swiglu_vec_kernel).
inline unsigned grid_for(int64_t work_items)
{
    const int64_t b = ceil_div(work_items, 256), most = (int64_t{1} << 31) - 1;
    return static_cast<unsigned>(b < 1 ? 1 : (b > most ? most : b));
}

template <typename T> int swiglu_impl(const void *X, int64_t R, int64_t D, float beta, void *Y, hipStream_t s)
{
    if (R == 0 || D == 0) return OPMX_OK;
    constexpr int n = Vec16<T>::n;
    const bool vec = D % n == 0 && aligned16(X) && aligned16(Y);
    const int64_t chunks = vec ? D / n : D;
    const dim3 grid(static_cast<unsigned>(ceil_div(chunks, 256)), static_cast<unsigned>(R < 65535 ? R : 65535));
    if (vec)
        swiglu_vec_kernel<T><<<grid, 256, 0, s>>>(static_cast<const T *>(X), R, D, beta, static_cast<T *>(Y));
    else
        swiglu_scalar_kernel<T><<<grid, 256, 0, s>>>(static_cast<const T *>(X), R, D, beta, static_cast<T *>(Y));
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T> int silu_impl(const void *X, const void *gate, int64_t cnt, void *Y, hipStream_t s)
{
    if (cnt == 0) return OPMX_OK;
    constexpr int n = Vec16<T>::n;
    const bool vec = cnt % n == 0 && aligned16(X) && aligned16(Y) && (!gate || aligned16(gate));
    if (vec)
        silu_kernel<T, true><<<grid_for(cnt / n), 256, 0, s>>>(static_cast<const T *>(X),
                                                              static_cast<const T *>(gate), cnt, static_cast<T *>(Y));
    else
        silu_kernel<T, false><<<grid_for(cnt), 256, 0, s>>>(static_cast<const T *>(X), static_cast<const T *>(gate),
                                                           cnt, static_cast<T *>(Y));
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

int launch_swiglu(const void *X, int64_t R, int64_t D, float beta, int dtype, void *Y, hipStream_t s)
{
    switch (dtype) {
        case OPMX_DTYPE_F32: return swiglu_impl<float>(X, R, D, beta, Y, s);
        case OPMX_DTYPE_F16: return swiglu_impl<f16>(X, R, D, beta, Y, s);
        case OPMX_DTYPE_BF16: return swiglu_impl<bf16>(X, R, D, beta, Y, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

int launch_silu(const void *X, const void *gate, int64_t n, int dtype, void *Y, hipStream_t s)
{
    switch (dtype) {
        case OPMX_DTYPE_F32: return silu_impl<float>(X, gate, n, Y, s);
        case OPMX_DTYPE_F16: return silu_impl<f16>(X, gate, n, Y, s);
        case OPMX_DTYPE_BF16: return silu_impl<bf16>(X, gate, n, Y, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
