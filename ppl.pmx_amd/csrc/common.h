// Shared device helpers for the OPMX MoE kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "opmx_moe.h"

namespace opmx {

using f16 = _Float16;
using bf16 = __bf16;

constexpr int kWave = 64;

template <typename T> struct DType;
template <> struct DType<float> { static constexpr int id = OPMX_DTYPE_F32; };
template <> struct DType<f16> { static constexpr int id = OPMX_DTYPE_F16; };
template <> struct DType<bf16> { static constexpr int id = OPMX_DTYPE_BF16; };

template <typename T> __device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }  // RNE

// 16-byte vector of T.
template <typename T> struct Vec16 {
    static constexpr int n = 16 / sizeof(T);
    T v[n];
};
template <typename T> __device__ __forceinline__ Vec16<T> load16(const T *p)
{
    Vec16<T> r;
    *reinterpret_cast<uint4 *>(&r) = *reinterpret_cast<const uint4 *>(p);
    return r;
}
template <typename T> __device__ __forceinline__ void store16(T *p, const Vec16<T> &r)
{
    *reinterpret_cast<uint4 *>(p) = *reinterpret_cast<const uint4 *>(&r);
}
// The same for data that is read once: a load the caches need not keep.
template <typename T> __device__ __forceinline__ Vec16<T> load16_once(const T *p)
{
    typedef uint32_t quad __attribute__((ext_vector_type(4)));
    Vec16<T> r;
    const quad q = __builtin_nontemporal_load(reinterpret_cast<const quad *>(p));
    __builtin_memcpy(&r, &q, 16);
    return r;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Butterfly sum over the 64 lanes of a wave; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, kWave);
    return v;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// Hardware exp2 / reciprocal (about 1 ulp each in fp32): for epilogues whose result is rounded
// to 16 bits anyway, where the accurate routine costs MFMA-idle time on every output tile.
__device__ __forceinline__ float sigmoid_fast_(float x)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896341f));
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- the little process-wide state the library keeps (all of it thread-safe) ----
// Tuning / test knobs (opmx_moe_set_option; initial values from the environment variables of the
// same names, read once).  -1 = automatic.  They select between kernels that compute the same
// thing, never results beyond accumulation order.
enum Option {
    kOptGemm = 0,        // OPMX_MOE_GEMM: 1 generic, 2 tiled, 3 stream
    kOptTiledVariant,    // OPMX_MOE_GEMM_TILED_VARIANT: 0..3
    kOptStreamVariant,   // OPMX_MOE_GEMM_STREAM_VARIANT: 0..5
    kOptGnx,             // OPMX_MOE_GEMM_GNX: tile order 0 / 4 / 8 / 16
    kOptStreamK,         // OPMX_MOE_GEMM_STREAMK: 0 never split the tail tiles over K, 2 whenever possible
    kOptPersist,         // OPMX_MOE_GEMM_PERSIST: 0 never the persistent form, 1 whenever possible
    kOptRouteIndexTokens,  // OPMX_MOE_ROUTE_INDEX_TOKENS: up to how many tokens (0 ... 64) the index form of router
                           // gate + MoeSelect runs as one launch of one block
    kOptF32Variant,        // OPMX_MOE_GEMM_F32_VARIANT: few rows per expert, fp32: 0 the 128-column tile form, 1 the form
                           // whose waves split K
    kNumOptions
};
int option(Option o);

constexpr int kMaxDevices = 64;
// The ordinal of the GPU that is current on this thread, or -1.
inline int current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
    return dev;
}
// Raises a kernel's dynamic shared-memory limit, once per GPU and kernel.  `done` is that kernel's
// own bit mask of the GPUs already served.  Two threads that arrive together both set the
// (same) attribute; neither launches before it is set.
inline bool ensure_dynamic_smem(const void *kernel, int bytes, std::atomic<uint64_t> &done)
{
    const int dev = current_device();
    if (dev < 0) return false;
    const uint64_t bit = uint64_t{1} << dev;
    if (done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    done.fetch_or(bit, std::memory_order_release);
    return true;
}
// Compute units of the current GPU (looked up once per GPU), 0 on failure.
int cu_count();

#define OPMX_LAUNCH_CHECK()                                   \
    do {                                                      \
        if (hipGetLastError() != hipSuccess) return OPMX_ERR_LAUNCH; \
    } while (0)

// Host launchers (one per translation unit); all return an opmx_status.
int launch_linear(const void *X, const void *W, const void *B, int64_t T, int64_t K, int64_t N,
                  int dtype, void *Y, hipStream_t s);
// Xp == nullptr: routing only (no row copy); row_token (may be nullptr) receives, for every row of the
// permuted order, the token whose copy it is.
int launch_linear_route(const void *X, const void *W, const void *B, int64_t T, int64_t K, int E, int k, int dtype,
                        void *scores, void *weights, int32_t *ids, hipStream_t s);
int launch_moe_select(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                      void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids, void *ws,
                      hipStream_t s, int32_t *row_token = nullptr);
size_t moe_select_workspace_bytes(int64_t T, int E, int k);
int launch_moe_select_static(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                             void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids, hipStream_t s);
int launch_moe_route_select(const void *X, const void *Wg, const void *Bg, int64_t T, int64_t H, int E, int k,
                            int dtype, void *scores, void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids,
                            void *ws, hipStream_t s, int32_t *row_token = nullptr);
int launch_swiglu(const void *X, int64_t R, int64_t D, float beta, int dtype, void *Y, hipStream_t s);
int launch_silu(const void *X, const void *gate, int64_t n, int dtype, void *Y, hipStream_t s);
int launch_rms_norm(const void *X, const void *Wt, const void *Skip, int64_t T, int64_t H, float eps, int dtype,
                    void *Y, void *SkipOut, hipStream_t s);
int launch_moe_reduce(const void *Y, const void *w, const int64_t *inv, int64_t T, int k, int64_t N,
                      int dtype, void *out, hipStream_t s);
size_t grouped_gemm_workspace_bytes(int E, int64_t R, int64_t K, int64_t N, int dtype);

}  // namespace opmx
