// SwiGLU and gated SiLU for gfx950 (elementwise, HBM bound, 16 bytes per lane).
// Semantics: torch_function/SwiGLU.py:15-16 and torch_function/SiLU.py:18-21.
#include "common.h"

namespace opmx {
namespace {

// Y[r,i] = (g * x) * sigmoid(beta*x), x = X[r,i], g = X[r,D+i]
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const T *__restrict__ X, int64_t R, int64_t D, float beta,
                                                     T *__restrict__ Y)
{
    constexpr int n = VEC ? Vec16<T>::n : 1;
    const int64_t per_row = D / n;
    const int64_t total = R * per_row;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t r = i / per_row, c = (i - r * per_row) * n;
        const T *px = X + r * 2 * D + c;
        if (VEC) {
            Vec16<T> x = load16(px), g = load16(px + D), o;
#pragma unroll
            for (int j = 0; j < n; ++j) {
                float xf = to_f32(x.v[j]), gf = to_f32(g.v[j]);
                o.v[j] = from_f32<T>(gf * xf * sigmoidf_(beta * xf));
            }
            store16(Y + r * D + c, o);
        } else {
            float xf = to_f32(px[0]), gf = to_f32(px[D]);
            Y[r * D + c] = from_f32<T>(gf * xf * sigmoidf_(beta * xf));
        }
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
                float y = xf * sigmoidf_(xf);
                o.v[j] = from_f32<T>(gate ? to_f32(g.v[j]) * y : y);
            }
            store16(Y + i * n, o);
        } else {
            float xf = to_f32(X[i]);
            float y = xf * sigmoidf_(xf);
            Y[i] = from_f32<T>(gate ? to_f32(gate[i]) * y : y);
        }
    }
}

inline unsigned grid_for(int64_t work_items)
{
    int64_t b = ceil_div(work_items, 256);
    return static_cast<unsigned>(b < 1 ? 1 : (b > 8192 ? 8192 : b));
}

template <typename T> int swiglu_impl(const void *X, int64_t R, int64_t D, float beta, void *Y, hipStream_t s)
{
    if (R == 0 || D == 0) return OPMX_OK;
    constexpr int n = Vec16<T>::n;
    const bool vec = D % n == 0 && aligned16(X) && aligned16(Y);
    if (vec)
        swiglu_kernel<T, true><<<grid_for(R * (D / n)), 256, 0, s>>>(static_cast<const T *>(X), R, D, beta,
                                                                    static_cast<T *>(Y));
    else
        swiglu_kernel<T, false><<<grid_for(R * D), 256, 0, s>>>(static_cast<const T *>(X), R, D, beta,
                                                               static_cast<T *>(Y));
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
