// Skinny linear for gfx950: Y = X W^T (+B) with few output features (the MoE
// router gate, N = number of experts).  HBM bound on X: every block streams its
// tokens' rows once with 16-byte loads and keeps W in cache.
// Semantics: torch_function/Linear.py:32 of OpenPPL/ppl.pmx.
#include "moe_gemm.h"
#include "moe_route.h"

namespace opmx {
namespace {

constexpr int kNT = 8;   // output features per pass

template <typename T, int TPB, bool VEC>
__global__ __launch_bounds__(256) void linear_kernel(const T *__restrict__ X, const T *__restrict__ W,
                                                     const T *__restrict__ B, int64_t Ttok, int64_t K, int64_t N,
                                                     T *__restrict__ Y)
{
    constexpr int n = VEC ? Vec16<T>::n : 1;
    __shared__ float red[256 / kWave][TPB * kNT];
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * TPB;
    const int lane = lane_id(), wave = threadIdx.x / kWave;

    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * kNT;   // one tile of kNT outputs per block
    float acc[TPB][kNT];
#pragma unroll
    for (int a = 0; a < TPB; ++a)
#pragma unroll
        for (int j = 0; j < kNT; ++j) acc[a][j] = 0.0f;

    for (int64_t c = static_cast<int64_t>(threadIdx.x) * n; c < K; c += 256 * n) {
        float xv[TPB][n];
#pragma unroll
        for (int a = 0; a < TPB; ++a) {
            const int64_t t = t0 + a < Ttok ? t0 + a : Ttok - 1;
            if (VEC) {
                Vec16<T> v = load16(X + t * K + c);
#pragma unroll
                for (int i = 0; i < n; ++i) xv[a][i] = to_f32(v.v[i]);
            } else {
                xv[a][0] = to_f32(X[t * K + c]);
            }
        }
#pragma unroll
        for (int j = 0; j < kNT; ++j) {
            const int64_t row = n0 + j < N ? n0 + j : N - 1;
            float wv[n];
            if (VEC) {
                Vec16<T> v = load16(W + row * K + c);
#pragma unroll
                for (int i = 0; i < n; ++i) wv[i] = to_f32(v.v[i]);
            } else {
                wv[0] = to_f32(W[row * K + c]);
            }
#pragma unroll
            for (int a = 0; a < TPB; ++a)
#pragma unroll
                for (int i = 0; i < n; ++i) acc[a][j] += xv[a][i] * wv[i];
        }
    }
#pragma unroll
    for (int a = 0; a < TPB; ++a)
#pragma unroll
        for (int j = 0; j < kNT; ++j) {
            float v = wave_sum(acc[a][j]);
            if (lane == 0) red[wave][a * kNT + j] = v;
        }
    __syncthreads();
    if (threadIdx.x < TPB * kNT) {
        const int a = threadIdx.x / kNT, j = threadIdx.x % kNT;
        if (t0 + a < Ttok && n0 + j < N) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < 256 / kWave; ++w) v += red[w][threadIdx.x];
            if (B) v += to_f32(B[n0 + j]);
            Y[(t0 + a) * N + n0 + j] = from_f32<T>(v);
        }
    }
}

// Many tokens, few outputs (the router gate of a long prompt), fp16/bf16: a block takes 16 tokens
// and all N <= 64 outputs, its NW waves split K (wave w takes the 32-wide k-steps w, w+NW, ...)
// and feed the MFMA 16x16x32 units straight from global memory: X is read once, 64-byte pieces
// of 16 rows per load with four steps in flight, W comes from cache.  The partial sums meet in
// LDS and are added in wave order.  NE = 16-output tiles per token tile.
// ROUTE: the block holds all N <= 64 logits of its 16 tokens (one block over the outputs), rounds
// them, and goes on to route those tokens on the rounded values -- top-k, ties to the lower expert
// id, softmax over the picks (MoeSelect.py:40-41) -- writing expert ids and weights next to the
// logits: MoeSelect then starts from the picks and the logits are never read back.
template <typename T, int NE, int NW, bool ROUTE>
__global__ __launch_bounds__(NW * 64) void linear_skinny_mfma_kernel(const T *__restrict__ X, const T *__restrict__ W,
                                                                      const T *__restrict__ B, int64_t Ttok, int64_t K,
                                                                      int64_t N, T *__restrict__ Y, int k,
                                                                      T *__restrict__ weights, int32_t *__restrict__ ids)
{
    using frag = typename Mfma<T>::frag;
    __shared__ __attribute__((aligned(16))) float part[NW * NE * 64 * 4];
    __shared__ T s_scores[ROUTE ? 16 * NE * 16 : 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fr = lane & 15, fg = lane >> 4;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * 16;
    const int64_t trow = t0 + fr < Ttok ? t0 + fr : Ttok - 1;      // rows past the end repeat the last one
    const T *xp = X + trow * K + fg * 8;
    const int64_t n0 = static_cast<int64_t>(blockIdx.y) * (NE * 16);   // this block's outputs: [n0, n0 + 16 NE)
    const T *wp[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        const int64_t n = n0 + e * 16 + fr < N ? n0 + e * 16 + fr : N - 1;
        wp[e] = W + n * K + fg * 8;
    }
    float4_t acc[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) acc[e] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int steps = static_cast<int>(K / 32);
    int st = wave;
    for (; st + 3 * NW < steps; st += 4 * NW) {
        frag b[4], a[4][NE];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            b[u] = __builtin_nontemporal_load(reinterpret_cast<const frag *>(xp + (st + NW * u) * 32));
#pragma unroll
            for (int e = 0; e < NE; ++e) a[u][e] = *reinterpret_cast<const frag *>(wp[e] + (st + NW * u) * 32);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < NE; ++e) acc[e] = Mfma<T>::m16(a[u][e], b[u], acc[e]);
    }
    for (; st < steps; st += NW) {
        const frag b = __builtin_nontemporal_load(reinterpret_cast<const frag *>(xp + st * 32));
#pragma unroll
        for (int e = 0; e < NE; ++e)
            acc[e] = Mfma<T>::m16(*reinterpret_cast<const frag *>(wp[e] + st * 32), b, acc[e]);
    }
    // acc[e][i]: output e*16 + fg*4 + i, token t0 + fr
#pragma unroll
    for (int e = 0; e < NE; ++e) *reinterpret_cast<float4_t *>(part + ((wave * NE + e) * 64 + lane) * 4) = acc[e];
    __syncthreads();
    for (int q = threadIdx.x; q < 16 * NE * 16; q += NW * 64) {
        const int t = q / (NE * 16), n = q % (NE * 16);
        if (t0 + t >= Ttok || n0 + n >= N) continue;
        const int idx = (((n >> 4) * 64) + (((n & 15) >> 2) * 16 + t)) * 4 + (n & 3);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) v += part[w * NE * 64 * 4 + idx];
        if (B) v += to_f32(B[n0 + n]);
        const T r = from_f32<T>(v);
        Y[(t0 + t) * N + n0 + n] = r;
        if (ROUTE) s_scores[t * static_cast<int>(N) + n] = r;
    }
    if (ROUTE) {
        __syncthreads();
        const int E = static_cast<int>(N);
        int G = 8;
        while (G < E) G <<= 1;                  // E <= 64: one key per lane
        const int lig = threadIdx.x % G, grp = threadIdx.x / G, ngrp = NW * 64 / G;
        for (int tl = grp; tl < 16; tl += ngrp) {            // whole lane groups iterate together
            if (t0 + tl >= Ttok) break;
            int id;
            float w;
            route_token(s_scores + tl * E, E, k, G, 1, lig, id, w);
            if (lig < k) {
                ids[(t0 + tl) * k + lig] = id;
                weights[(t0 + tl) * k + lig] = from_f32<T>(w);
            }
        }
    }
}

template <typename T>
int linear_skinny_mfma(const void *X, const void *W, const void *B, int64_t Ttok, int64_t K, int64_t N, void *Y,
                       hipStream_t s)
{
    constexpr int NW = 8;
    const unsigned grid = static_cast<unsigned>(ceil_div(Ttok, 16));
    const T *x = static_cast<const T *>(X), *w = static_cast<const T *>(W), *b = static_cast<const T *>(B);
    T *y = static_cast<T *>(Y);
    if (N <= 16) linear_skinny_mfma_kernel<T, 1, NW, false><<<grid, NW * 64, 0, s>>>(x, w, b, Ttok, K, N, y, 0, nullptr, nullptr);
    else if (N <= 32) linear_skinny_mfma_kernel<T, 2, NW, false><<<grid, NW * 64, 0, s>>>(x, w, b, Ttok, K, N, y, 0, nullptr, nullptr);
    else   // 64 outputs per block; more outputs: more blocks over the same tokens (X read once per 64 outputs)
        linear_skinny_mfma_kernel<T, 4, NW, false><<<dim3(grid, static_cast<unsigned>(ceil_div(N, 64))), NW * 64, 0, s>>>(
            x, w, b, Ttok, K, N, y, 0, nullptr, nullptr);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

// The same kernel with the routing of its tokens in the epilogue (N = number of experts <= 64).
template <typename T>
int linear_skinny_route(const void *X, const void *W, const void *B, int64_t Ttok, int64_t K, int64_t N, int k, void *Y,
                        void *weights, int32_t *ids, hipStream_t s)
{
    constexpr int NW = 8;
    const unsigned grid = static_cast<unsigned>(ceil_div(Ttok, 16));
    const T *x = static_cast<const T *>(X), *w = static_cast<const T *>(W), *b = static_cast<const T *>(B);
    T *y = static_cast<T *>(Y), *wt = static_cast<T *>(weights);
    if (N <= 16) linear_skinny_mfma_kernel<T, 1, NW, true><<<grid, NW * 64, 0, s>>>(x, w, b, Ttok, K, N, y, k, wt, ids);
    else if (N <= 32) linear_skinny_mfma_kernel<T, 2, NW, true><<<grid, NW * 64, 0, s>>>(x, w, b, Ttok, K, N, y, k, wt, ids);
    else linear_skinny_mfma_kernel<T, 4, NW, true><<<grid, NW * 64, 0, s>>>(x, w, b, Ttok, K, N, y, k, wt, ids);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T>
int linear_impl(const void *X_, const void *W_, const void *B_, int64_t Ttok, int64_t K, int64_t N, void *Y_,
                hipStream_t s)
{
    if (Ttok == 0 || N == 0) return OPMX_OK;
    const T *X = static_cast<const T *>(X_), *W = static_cast<const T *>(W_), *B = static_cast<const T *>(B_);
    T *Y = static_cast<T *>(Y_);
    const bool vec = K % Vec16<T>::n == 0 && aligned16(X) && aligned16(W);
    if (Ttok >= 4096) {
        // 8 tokens per block: W (read from cache by every block) is amortised over more rows of X
        const dim3 grid(static_cast<unsigned>(ceil_div(Ttok, 8)), static_cast<unsigned>(ceil_div(N, kNT)));
        if (vec) linear_kernel<T, 8, true><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
        else linear_kernel<T, 8, false><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
    } else if (Ttok >= 1024) {
        const dim3 grid(static_cast<unsigned>(ceil_div(Ttok, 4)), static_cast<unsigned>(ceil_div(N, kNT)));
        if (vec) linear_kernel<T, 4, true><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
        else linear_kernel<T, 4, false><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
    } else {
        const dim3 grid(static_cast<unsigned>(Ttok), static_cast<unsigned>(ceil_div(N, kNT)));
        if (vec) linear_kernel<T, 1, true><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
        else linear_kernel<T, 1, false><<<grid, 256, 0, s>>>(X, W, B, Ttok, K, N, Y);
    }
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

// Whether the router logits of T tokens over N experts go through linear_skinny_mfma_kernel
// (measured crossovers against the other two kernels, see launch_linear).
static bool skinny_mfma_pays(int64_t T, int64_t K, int64_t N, int dtype, const void *X, const void *W)
{
    return (dtype == OPMX_DTYPE_F16 || dtype == OPMX_DTYPE_BF16) && N <= 256 && K >= 32 && K % 32 == 0 && aligned16(X) &&
           aligned16(W) &&
           (N <= 8 ? T >= 4096 : N <= 64 ? (T >= 512 && (N <= 16 || T < 8192)) : (T * N >= 32768 && T * N <= 262144));
}

// Router logits and, in the same launch, the routing of every token on them: scores [T,E] as
// launch_linear writes them, expert ids [T,k] and weights [T,k] as MoeSelect's top-k kernel writes
// them.  Only where the skinny MFMA kernel is the router kernel anyway and one block holds a
// token's E <= 64 logits; OPMX_ERR_UNSUPPORTED otherwise (nothing enqueued: the caller runs the
// two operators one after the other).
int launch_linear_route(const void *X, const void *W, const void *B, int64_t T, int64_t K, int E, int k, int dtype,
                        void *scores, void *weights, int32_t *ids, hipStream_t s)
{
    if (E > 64 || k > E || !skinny_mfma_pays(T, K, E, dtype, X, W)) return OPMX_ERR_UNSUPPORTED;
    return dtype == OPMX_DTYPE_F16 ? linear_skinny_route<f16>(X, W, B, T, K, E, k, scores, weights, ids, s)
                                   : linear_skinny_route<bf16>(X, W, B, T, K, E, k, scores, weights, ids, s);
}

int launch_linear(const void *X, const void *W, const void *B, int64_t T, int64_t K, int64_t N, int dtype,
                  void *Y, hipStream_t s)
{
    // Many tokens: the MFMA tile kernel in dense mode (no expert_offset: one segment [0,T))
    // reads X once with 128x128 tiles instead of one pass per 8 output features.
    // Few outputs, many tokens: the MFMA kernel that splits K over the waves of a block.  Measured
    // against the other two (H = 4096, 8 outputs: 10 us against 19 at T = 4096, 18 against 30 at
    // 8192, no gain below; H = 2048, 64 outputs: 12-13 us against the tile kernel's 21 from T = 512
    // to 4096, while from 8192 tokens on the tile kernel re-reads W less and wins; H = 7168, 256 outputs
    // in four blocks of 64 over the same tokens: 37 us against 64 up to T = 1024, 71 against 64 at 2048;
    // its K chain costs about H / 195 us whatever T is, which one block per token undercuts up to
    // T * N of about 32768: 256 outputs, T = 128: 31 us per-token blocks, 36 us this kernel; T = 256: 61 / 37).
    if (skinny_mfma_pays(T, K, N, dtype, X, W))
        return dtype == OPMX_DTYPE_F16 ? linear_skinny_mfma<f16>(X, W, B, T, K, N, Y, s)
                                       : linear_skinny_mfma<bf16>(X, W, B, T, K, N, Y, s);
    if ((dtype == OPMX_DTYPE_F16 || dtype == OPMX_DTYPE_BF16) && T >= 512 && N > 8 && K % 64 == 0 &&
        aligned16(X) && aligned16(W) && N * K < (int64_t{1} << 31))
        return launch_gemm_tiled(X, nullptr, W, B, 1, T, K, N, dtype, OPMX_EPILOGUE_NONE, /*128x128 tiles*/ 2, Y, nullptr, 0, s);
    switch (dtype) {
        case OPMX_DTYPE_F32: return linear_impl<float>(X, W, B, T, K, N, Y, s);
        case OPMX_DTYPE_F16: return linear_impl<f16>(X, W, B, T, K, N, Y, s);
        case OPMX_DTYPE_BF16: return linear_impl<bf16>(X, W, B, T, K, N, Y, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
