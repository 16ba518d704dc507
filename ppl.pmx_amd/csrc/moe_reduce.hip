// MoeReduce for gfx950: out[t] = sum_s w[t,s] * Y[inv[t,s]], the gather, the
// expert weighting and the sum fused in one pass (fp32, one rounding).
// Semantics: torch_function/MoeReduce.py:23-25 of OpenPPL/ppl.pmx.
#include "common.h"

namespace opmx {
namespace {

constexpr int kMaxK = OPMX_MOE_MAX_EXPERTS_PER_TOKEN;

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void moe_reduce_kernel(const T *__restrict__ Y, const T *__restrict__ w,
                                                         const int64_t *__restrict__ inv, int64_t Ttok, int k,
                                                         int64_t N, int64_t R, T *__restrict__ out)
{
    __shared__ float sw[kMaxK];
    __shared__ int64_t srow[kMaxK];
    for (int64_t t = blockIdx.x; t < Ttok; t += gridDim.x) {
        __syncthreads();
        if (threadIdx.x < k) {
            sw[threadIdx.x] = to_f32(w[t * k + threadIdx.x]);
            int64_t r = inv[t * k + threadIdx.x];
            srow[threadIdx.x] = r < 0 ? 0 : (r >= R ? R - 1 : r);   // never read outside Y
        }
        __syncthreads();
        if (VEC) {
            constexpr int n = Vec16<T>::n;
            for (int64_t c = static_cast<int64_t>(threadIdx.x) * n; c < N; c += static_cast<int64_t>(blockDim.x) * n) {
                float acc[n];
#pragma unroll
                for (int i = 0; i < n; ++i) acc[i] = 0.0f;
                int s = 0;
                for (; s + 4 <= k; s += 4) {       // four gathered rows in flight; summed in slot order
                    Vec16<T> v[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) v[u] = load16(Y + srow[s + u] * N + c);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float ws = sw[s + u];
#pragma unroll
                        for (int i = 0; i < n; ++i) acc[i] += ws * to_f32(v[u].v[i]);
                    }
                }
                for (; s < k; ++s) {
                    Vec16<T> v = load16(Y + srow[s] * N + c);
                    float ws = sw[s];
#pragma unroll
                    for (int i = 0; i < n; ++i) acc[i] += ws * to_f32(v.v[i]);
                }
                Vec16<T> o;
#pragma unroll
                for (int i = 0; i < n; ++i) o.v[i] = from_f32<T>(acc[i]);
                store16(out + t * N + c, o);
            }
        } else {
            for (int64_t c = threadIdx.x; c < N; c += blockDim.x) {
                float acc = 0.0f;
                for (int s = 0; s < k; ++s) acc += sw[s] * to_f32(Y[srow[s] * N + c]);
                out[t * N + c] = from_f32<T>(acc);
            }
        }
    }
}

template <typename T>
int reduce_impl(const void *Y, const void *w, const int64_t *inv, int64_t Ttok, int k, int64_t N, void *out,
                hipStream_t s)
{
    if (Ttok == 0 || N == 0) return OPMX_OK;
    const bool vec = (N * sizeof(T)) % 16 == 0 && aligned16(Y) && aligned16(out);
    const unsigned grid = static_cast<unsigned>(Ttok < 65536 ? Ttok : 65536);
    if (vec)
        moe_reduce_kernel<T, true><<<grid, 256, 0, s>>>(static_cast<const T *>(Y), static_cast<const T *>(w), inv,
                                                        Ttok, k, N, Ttok * k, static_cast<T *>(out));
    else
        moe_reduce_kernel<T, false><<<grid, 256, 0, s>>>(static_cast<const T *>(Y), static_cast<const T *>(w), inv,
                                                         Ttok, k, N, Ttok * k, static_cast<T *>(out));
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

int launch_moe_reduce(const void *Y, const void *w, const int64_t *inv, int64_t T, int k, int64_t N, int dtype,
                      void *out, hipStream_t s)
{
    switch (dtype) {
        case OPMX_DTYPE_F32: return reduce_impl<float>(Y, w, inv, T, k, N, out, s);
        case OPMX_DTYPE_F16: return reduce_impl<f16>(Y, w, inv, T, k, N, out, s);
        case OPMX_DTYPE_BF16: return reduce_impl<bf16>(Y, w, inv, T, k, N, out, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
