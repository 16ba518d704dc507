// RMSNorm / SkipRMSNorm for gfx950: the operator directly in front of the MoE layer (ffn_norm).
// HBM bound: every row is read once (X and the skip input), kept in registers, and written once
// (Y and the skip output).
// Semantics, with the roundings of torch_function/RMSNorm.py:16-24 and :44-56:
//   s    = round_T(X + SkipIn)            (s = X without a skip input)
//   y    = float(s) * rsqrt(mean(float(s)^2) + eps)
//   Y    = round_T(round_T(y) * weight)   (the reference rounds y to T before the multiply)
//   SkipOut = s
#include "common.h"

namespace opmx {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ float block_sum(float v, float *red)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < kThreads / 64; ++w) t += red[w];
    __syncthreads();
    return t;
}

// One block per row; a thread owns CH 16-byte chunks of the row (chunk c of thread t is element
// (c*kThreads + t) * n), kept in registers between the two passes.  H % n == 0, H <= CH*kThreads*n.
template <typename T, int CH>
__global__ __launch_bounds__(kThreads) void rms_norm_kernel(const T *__restrict__ X, const T *__restrict__ Wt,
                                                            const T *__restrict__ Skip, int64_t H, float eps,
                                                            T *__restrict__ Y, T *__restrict__ SkipOut)
{
    constexpr int n = Vec16<T>::n;
    __shared__ float red[kThreads / 64];
    const int64_t row = blockIdx.x;
    const T *x = X + row * H;
    const T *sk = Skip ? Skip + row * H : nullptr;
    Vec16<T> s[CH];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int64_t e = (static_cast<int64_t>(c) * kThreads + threadIdx.x) * n;
        if (e < H) {
            s[c] = load16(x + e);
            if (sk) {
                const Vec16<T> k = load16(sk + e);
#pragma unroll
                for (int j = 0; j < n; ++j) s[c].v[j] = from_f32<T>(to_f32(s[c].v[j]) + to_f32(k.v[j]));
            }
#pragma unroll
            for (int j = 0; j < n; ++j) {
                const float f = to_f32(s[c].v[j]);
                ss += f * f;
            }
            if (SkipOut) store16(SkipOut + row * H + e, s[c]);
        }
    }
    const float scale = rsqrtf(block_sum(ss, red) / static_cast<float>(H) + eps);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int64_t e = (static_cast<int64_t>(c) * kThreads + threadIdx.x) * n;
        if (e < H) {
            const Vec16<T> w = load16(Wt + e);
            Vec16<T> o;
#pragma unroll
            for (int j = 0; j < n; ++j)
                o.v[j] = from_f32<T>(to_f32(from_f32<T>(to_f32(s[c].v[j]) * scale)) * to_f32(w.v[j]));
            store16(Y + row * H + e, o);
        }
    }
}

// Any H and alignment: element-wise, the row is read twice.
template <typename T>
__global__ __launch_bounds__(kThreads) void rms_norm_generic_kernel(const T *__restrict__ X, const T *__restrict__ Wt,
                                                                    const T *__restrict__ Skip, int64_t H, float eps,
                                                                    T *__restrict__ Y, T *__restrict__ SkipOut)
{
    __shared__ float red[kThreads / 64];
    const int64_t row = blockIdx.x;
    float ss = 0.0f;
    for (int64_t e = threadIdx.x; e < H; e += kThreads) {
        T s = X[row * H + e];
        if (Skip) s = from_f32<T>(to_f32(s) + to_f32(Skip[row * H + e]));
        const float f = to_f32(s);
        ss += f * f;
        if (SkipOut) SkipOut[row * H + e] = s;
    }
    const float scale = rsqrtf(block_sum(ss, red) / static_cast<float>(H) + eps);
    for (int64_t e = threadIdx.x; e < H; e += kThreads) {
        T s = X[row * H + e];
        if (Skip) s = from_f32<T>(to_f32(s) + to_f32(Skip[row * H + e]));
        Y[row * H + e] = from_f32<T>(to_f32(from_f32<T>(to_f32(s) * scale)) * to_f32(Wt[e]));
    }
}

template <typename T>
int rms_norm_impl(const void *X, const void *Wt, const void *Skip, int64_t T_, int64_t H, float eps, void *Y,
                  void *SkipOut, hipStream_t s)
{
    constexpr int n = Vec16<T>::n;
    const T *x = static_cast<const T *>(X), *w = static_cast<const T *>(Wt), *k = static_cast<const T *>(Skip);
    T *y = static_cast<T *>(Y), *so = static_cast<T *>(SkipOut);
    const bool vec = H % n == 0 && aligned16(X) && aligned16(Wt) && aligned16(Y) && (!Skip || aligned16(Skip)) &&
                     (!SkipOut || aligned16(SkipOut));
    const int64_t chunks = vec ? ceil_div(H / n, kThreads) : 0;
    dim3 grid(static_cast<unsigned>(T_)), block(kThreads);
    if (vec && chunks <= 1) rms_norm_kernel<T, 1><<<grid, block, 0, s>>>(x, w, k, H, eps, y, so);
    else if (vec && chunks <= 2) rms_norm_kernel<T, 2><<<grid, block, 0, s>>>(x, w, k, H, eps, y, so);
    else if (vec && chunks <= 4) rms_norm_kernel<T, 4><<<grid, block, 0, s>>>(x, w, k, H, eps, y, so);
    else if (vec && chunks <= 8) rms_norm_kernel<T, 8><<<grid, block, 0, s>>>(x, w, k, H, eps, y, so);
    else rms_norm_generic_kernel<T><<<grid, block, 0, s>>>(x, w, k, H, eps, y, so);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

int launch_rms_norm(const void *X, const void *Wt, const void *Skip, int64_t T, int64_t H, float eps, int dtype,
                    void *Y, void *SkipOut, hipStream_t s)
{
    if (T == 0 || H == 0) return OPMX_OK;
    if (T >= (int64_t{1} << 31)) return OPMX_ERR_UNSUPPORTED;
    switch (dtype) {
        case OPMX_DTYPE_F32: return rms_norm_impl<float>(X, Wt, Skip, T, H, eps, Y, SkipOut, s);
        case OPMX_DTYPE_F16: return rms_norm_impl<f16>(X, Wt, Skip, T, H, eps, Y, SkipOut, s);
        case OPMX_DTYPE_BF16: return rms_norm_impl<bf16>(X, Wt, Skip, T, H, eps, Y, SkipOut, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
