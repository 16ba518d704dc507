// SwiGLU and gated SiLU for gfx950 (elementwise, HBM bound, 16 bytes per lane).
// Semantics: torch_function/SwiGLU.py:15-16 and torch_function/SiLU.py:18-21.
#include "common.h"

namespace opmx {
namespace {

// Y[r,i] = (g * x) * sigmoid(beta*x), x = X[r,i], g = X[r,D+i].  A thread owns one 16-byte
// column chunk (blockIdx.x) and walks rows blockIdx.y, blockIdx.y + gridDim.y, ..., two rows per
// step so that four loads are in flight: no index division, coalesced along the row.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const T *__restrict__ X, int64_t R, int64_t D, float beta,
                                                     T *__restrict__ Y)
{
    constexpr int n = VEC ? Vec16<T>::n : 1;
    const int64_t c = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * n;
    if (c >= D) return;
    const int64_t step = gridDim.y;
    int64_t r = blockIdx.y;
    if (VEC) {
        for (; r + step < R; r += 2 * step) {
            const T *p0 = X + r * 2 * D + c, *p1 = X + (r + step) * 2 * D + c;
            Vec16<T> x0 = load16_once(p0), g0 = load16_once(p0 + D), x1 = load16_once(p1), g1 = load16_once(p1 + D), o0, o1;
#pragma unroll
            for (int j = 0; j < n; ++j) {
                const float a = to_f32(x0.v[j]), b = to_f32(x1.v[j]);
                o0.v[j] = from_f32<T>(to_f32(g0.v[j]) * a * sigmoidf_(beta * a));
                o1.v[j] = from_f32<T>(to_f32(g1.v[j]) * b * sigmoidf_(beta * b));
            }
            store16(Y + r * D + c, o0);
            store16(Y + (r + step) * D + c, o1);
        }
    }
    for (; r < R; r += step) {
        const T *px = X + r * 2 * D + c;
        if (VEC) {
            Vec16<T> x = load16_once(px), g = load16_once(px + D), o;
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
    // columns over x; rows over y, as many row lanes as it takes to have ~16 blocks per CU
    const int64_t chunks = vec ? D / n : D;
    const unsigned gx = static_cast<unsigned>(ceil_div(chunks, 256));
    int64_t gy = ceil_div(4096, gx);
    if (gy > R) gy = R;
    if (gy > 65535) gy = 65535;
    const dim3 grid(gx, static_cast<unsigned>(gy));
    if (vec)
        swiglu_kernel<T, true><<<grid, 256, 0, s>>>(static_cast<const T *>(X), R, D, beta, static_cast<T *>(Y));
    else
        swiglu_kernel<T, false><<<grid, 256, 0, s>>>(static_cast<const T *>(X), R, D, beta, static_cast<T *>(Y));
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
