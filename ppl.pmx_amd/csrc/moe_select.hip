// MoeSelect for gfx950: top-k with ties to the lower expert id, softmax over the
// picks, deterministic stable permutation by expert id, row expand/permute.
// Semantics: torch_function/MoeSelect.py:37-64 of OpenPPL/ppl.pmx.
//
// Determinism: positions never come from an atomic counter.  A token's row is
//   expert_offset[e] + (#tokens before it that picked e)
// and the count is taken from bit matrices (one bit per (expert, token)), whose
// construction by atomicOr is order independent.
#include <mutex>

#include "moe_gemm.h"
#include "moe_route.h"

namespace opmx {
namespace {

constexpr int kChunk = 256;          // tokens per routing block
constexpr int kWords = kChunk / 32;  // bit-matrix words per expert
__device__ __forceinline__ void zero_bits(uint32_t *bits, int E)
{
    for (int i = threadIdx.x; i < E * kWords; i += blockDim.x) bits[i] = 0u;
}

// rank of token `tl` (chunk-local) among the chunk's tokens that picked e
__device__ __forceinline__ int rank_in_chunk(const uint32_t *bits, const int *wordpre, int e, int tl)
{
    int w = tl >> 5;
    return wordpre[e * kWords + w] + __popc(bits[e * kWords + w] & ((1u << (tl & 31)) - 1u));
}

// per expert: exclusive prefix of the word popcounts; returns nothing, fills
// wordpre[e][w] and count[e]
__device__ __forceinline__ void word_prefix(const uint32_t *bits, int *wordpre, int *count, int E)
{
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < kWords; ++w) {
            wordpre[e * kWords + w] = run;
            run += __popc(bits[e * kWords + w]);
        }
        count[e] = run;
    }
}

// ---- general path, kernel 1: top-k + weights; one token per lane group ----
template <typename T>
__global__ __launch_bounds__(kChunk) void select_topk_kernel(const T *__restrict__ scores, int64_t Ttok,
                                                             int E, int k, int G, int vpl,
                                                             T *__restrict__ weights,
                                                             int32_t *__restrict__ ids)
{
    const int lig = threadIdx.x % G, grp = threadIdx.x / G, ngrp = kChunk / G;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * ngrp + grp;
    if (t >= Ttok) return;                 // whole lane groups leave together
    int id;
    float w;
    route_token(scores + t * E, E, k, G, vpl, lig, id, w);
    if (lig < k) {
        ids[t * k + lig] = id;
        weights[t * k + lig] = from_f32<T>(w);
    }
}

// ---- kernel 1b: per-chunk (256 tokens) expert histogram from the picked ids ----
__global__ __launch_bounds__(kChunk) void select_hist_kernel(const int32_t *__restrict__ ids, int64_t Ttok,
                                                             int E, int k, int32_t *__restrict__ hist)
{
    __shared__ uint32_t bits[OPMX_MOE_MAX_EXPERTS * kWords];
    const int tl = threadIdx.x;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kChunk + tl;
    zero_bits(bits, E);
    __syncthreads();
    if (t < Ttok)
        for (int s = 0; s < k; ++s) atomicOr(&bits[ids[t * k + s] * kWords + (tl >> 5)], 1u << (tl & 31));
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        int c = 0;
#pragma unroll
        for (int w = 0; w < kWords; ++w) c += __popc(bits[e * kWords + w]);
        hist[static_cast<int64_t>(blockIdx.x) * E + e] = c;
    }
}

// Exclusive scan of count[0..E) in place, total to count[E]; called by the first wave of a block
// (E <= 256: four experts per lane).  A single thread walking the experts costs two dependent LDS
// round trips per expert: 6 us for 64 experts, more than the rest of the small-T kernel.
__device__ __forceinline__ void scan_experts(int *count, int E)
{
    static_assert(OPMX_MOE_MAX_EXPERTS <= 4 * kWave, "four experts per lane");
    const int lane = lane_id();
    int v[4], tot = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane * 4 + j;
        v[j] = e < E ? count[e] : 0;
        tot += v[j];
    }
    int incl = tot;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += o;
    }
    int run = incl - tot;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane * 4 + j;
        if (e < E) count[e] = run;
        run += v[j];
    }
    if (lane == kWave - 1) count[E] = incl;
}

// ---- kernel 2: per expert exclusive scan over chunks, then offsets over experts ----
// One block; a wave scans one expert at a time (each a chain of dependent loads), so many
// experts get a block of 16 waves.
__global__ __launch_bounds__(1024) void select_scan_kernel(int32_t *__restrict__ hist, int nchunks, int E,
                                                           int64_t R, int64_t *__restrict__ off)
{
    __shared__ int total[OPMX_MOE_MAX_EXPERTS + 1];
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    for (int e = wave; e < E; e += static_cast<int>(blockDim.x) / kWave) {
        int running = 0;
        for (int c0 = 0; c0 < nchunks; c0 += kWave) {
            int c = c0 + lane;
            int v = c < nchunks ? hist[static_cast<int64_t>(c) * E + e] : 0;
            int incl = v;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                int o = __shfl_up(incl, d, kWave);
                if (lane >= d) incl += o;
            }
            if (c < nchunks) hist[static_cast<int64_t>(c) * E + e] = running + incl - v;
            running += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) total[e] = running;
    }
    __syncthreads();
    if (threadIdx.x < kWave) scan_experts(total, E);
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) off[e] = total[e];   // MoeSelect.py:54-59
    if (threadIdx.x == 0) off[E] = R;                                      // MoeSelect.py:60
}

// ---- kernel 3: rank inside the chunk -> invert_permutation ----
__global__ __launch_bounds__(kChunk) void select_rank_kernel(const int32_t *__restrict__ ids,
                                                             const int32_t *__restrict__ base,
                                                             const int64_t *__restrict__ off, int64_t Ttok,
                                                             int E, int k, int64_t *__restrict__ inv,
                                                             int32_t *__restrict__ row_token)
{
    __shared__ uint32_t bits[OPMX_MOE_MAX_EXPERTS * kWords];
    __shared__ int wordpre[OPMX_MOE_MAX_EXPERTS * kWords];
    __shared__ int count[OPMX_MOE_MAX_EXPERTS];
    const int tl = threadIdx.x;
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kChunk + tl;
    zero_bits(bits, E);
    __syncthreads();
    if (t < Ttok)
        for (int s = 0; s < k; ++s) atomicOr(&bits[ids[t * k + s] * kWords + (tl >> 5)], 1u << (tl & 31));
    __syncthreads();
    word_prefix(bits, wordpre, count, E);
    __syncthreads();
    if (t < Ttok)
        for (int s = 0; s < k; ++s) {
            int e = ids[t * k + s];
            const int64_t pos = off[e] + base[static_cast<int64_t>(blockIdx.x) * E + e] + rank_in_chunk(bits, wordpre, e, tl);
            inv[t * k + s] = pos;
            if (row_token) row_token[pos] = static_cast<int32_t>(t);   // the token whose copy row `pos` is (perm[pos] / k)
        }
}

// copy row X[t] to the k rows inv[t*k+s] of Xp
template <typename T>
__device__ __forceinline__ void expand_row(const T *__restrict__ X, T *__restrict__ Xp, int64_t t, int64_t H,
                                           int k, const int64_t *inv_row, bool vec)
{
    const T *src = X + t * H;
    if (vec) {
        constexpr int n = Vec16<T>::n;
        for (int64_t c = static_cast<int64_t>(threadIdx.x) * n; c < H; c += static_cast<int64_t>(blockDim.x) * n) {
            Vec16<T> v = load16(src + c);
            for (int s = 0; s < k; ++s) store16(Xp + inv_row[s] * H + c, v);
        }
    } else {
        for (int64_t c = threadIdx.x; c < H; c += blockDim.x) {
            T v = src[c];
            for (int s = 0; s < k; ++s) Xp[inv_row[s] * H + c] = v;
        }
    }
}

// ---- kernel 4: X_expand_permute[inv[t,s]] = X[t]  (MoeSelect.py:45-47) ----
template <typename T>
__global__ __launch_bounds__(256) void select_expand_kernel(const T *__restrict__ X, T *__restrict__ Xp,
                                                            const int64_t *__restrict__ inv, int64_t Ttok,
                                                            int64_t H, int k, bool vec)
{
    for (int64_t t = blockIdx.x; t < Ttok; t += gridDim.x) expand_row(X, Xp, t, H, k, inv + t * k, vec);
}

// Router logits of up to kFusedTokens tokens and kFusedExperts experts, computed by one
// 1024-thread block into LDS: scores[t][e] = X[t] . Wg[e] (+ Bg[e]), fp32 accumulation on the MFMA
// 16x16x32 units, rounded once to T (Linear.py:32).  The sixteen waves split K (a wave's few
// k-steps are in flight together: the phase costs about one memory round trip); their partial
// sums meet in LDS and are added in wave order, so the result does not depend on timing.  Every
// block of the fused kernel computes all logits redundantly, which is what lets one launch do
// router gate and routing without a grid-wide exchange -- and what limits it to few tokens.
// Measured on the Mixtral shape: one launch saves 1 us per layer at T = 1, breaks even at T = 8,
// costs 1-2 us at T = 16 (3-4 us with H = 6144) and 4.5 us at T = 32 (a two-tile form): a
// dependent launch on the same stream is cheap here, recomputing the logits per block is not.
// So one launch serves up to kFusedMaxTokens tokens; more go to the two separate kernels.
constexpr int kFusedTokens = 16, kFusedExperts = 16, kFusedWaves = 16;   // what the kernel can do
constexpr int kFusedMaxTokens = 8;                                       // what it is used for
template <typename T>
__device__ __forceinline__ void router_logits_to_lds(const T *__restrict__ X, const T *__restrict__ Wg,
                                                     const T *__restrict__ Bg, int Ttok, int64_t H, int E,
                                                     float *part /* [kFusedWaves][64][4] */, T *s_scores /* [Ttok*E] */)
{
    using frag = typename Mfma<T>::frag;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fr = lane & 15, fg = lane >> 4;
    const int erow = fr < E ? fr : E - 1;               // padded expert rows repeat the last one
    const int trow = fr < Ttok ? fr : Ttok - 1;         // padded token rows likewise
    const T *wp = Wg + static_cast<int64_t>(erow) * H + fg * 8;
    const T *xp = X + static_cast<int64_t>(trow) * H + fg * 8;
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    const int steps = static_cast<int>(H / 32);
    int st = wave;                      // wave w takes k-steps w, w+16, ... in this order
    for (; st + 3 * kFusedWaves < steps; st += 4 * kFusedWaves) {   // four steps' loads in flight
        frag a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            a[u] = *reinterpret_cast<const frag *>(wp + (st + kFusedWaves * u) * 32);
            b[u] = *reinterpret_cast<const frag *>(xp + (st + kFusedWaves * u) * 32);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) acc = Mfma<T>::m16(a[u], b[u], acc);
    }
    for (; st < steps; st += kFusedWaves) {
        const frag a = *reinterpret_cast<const frag *>(wp + st * 32);
        const frag b = *reinterpret_cast<const frag *>(xp + st * 32);
        acc = Mfma<T>::m16(a, b, acc);
    }
    // acc[i]: expert fg*4 + i, token fr
    *reinterpret_cast<float4_t *>(part + (wave * 64 + lane) * 4) = acc;
    __syncthreads();
    for (int q = threadIdx.x; q < Ttok * E; q += blockDim.x) {
        const int t = q / E, e = q % E;
        const int idx = ((e >> 2) * 16 + t) * 4 + (e & 3);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kFusedWaves; ++w) v += part[w * 64 * 4 + idx];
        if (Bg) v += to_f32(Bg[e]);
        s_scores[q] = from_f32<T>(v);
    }
    __syncthreads();
}

// ---- small-T path: one launch.  Every block routes all T <= kChunk tokens
// redundantly in LDS, then block b emits the outputs of token b and copies its row.
// With scores == nullptr the picks are read from ids_out instead (two-launch form: the routing
// work, T times redundant here, is what makes the one-launch form slow beyond a few tokens).
// FUSED: the router logits are computed here as well (scores = X Wg^T + Bg, T <= kFusedTokens,
// E <= kFusedExperts, 1024 threads) and written to `scores_out`, each block its own token's row.
template <typename T, bool FUSED>
__global__ __launch_bounds__(1024) void select_small_kernel(const T *__restrict__ X,
                                                              const T *__restrict__ scores, int Ttok,
                                                              int64_t H, int E, int k, int G, int vpl,
                                                              T *__restrict__ Xp, T *__restrict__ weights,
                                                              int64_t *__restrict__ inv,
                                                              int64_t *__restrict__ off,
                                                              int32_t *__restrict__ ids_out, bool vec,
                                                              const T *__restrict__ Wg, const T *__restrict__ Bg,
                                                              T *__restrict__ scores_out,
                                                              int32_t *__restrict__ row_token)
{
    __shared__ uint32_t bits[OPMX_MOE_MAX_EXPERTS * kWords];
    __shared__ int wordpre[OPMX_MOE_MAX_EXPERTS * kWords];
    __shared__ int count[OPMX_MOE_MAX_EXPERTS + 1];
    __shared__ int my_ids[OPMX_MOE_MAX_EXPERTS_PER_TOKEN];
    __shared__ int64_t my_inv[OPMX_MOE_MAX_EXPERTS_PER_TOKEN];
    __shared__ __attribute__((aligned(16))) float part[FUSED ? kFusedWaves * 64 * 4 : 4];
    __shared__ T s_scores[FUSED ? kFusedTokens * kFusedExperts : 1];
    const int lig = threadIdx.x % G, grp = threadIdx.x / G, ngrp = blockDim.x / G;
    const int me = blockIdx.x;                 // the token this block emits
    if constexpr (FUSED) {
        if constexpr (sizeof(T) == 2) router_logits_to_lds<T>(X, Wg, Bg, Ttok, H, E, part, s_scores);
        for (int e = threadIdx.x; e < E; e += blockDim.x) scores_out[static_cast<int64_t>(me) * E + e] = s_scores[me * E + e];
        scores = s_scores;
    }
    zero_bits(bits, E);
    __syncthreads();
    const bool picked = !FUSED && scores == nullptr;
    if (picked) {
        // the picks were made by select_topk_kernel (weights written there): only the bookkeeping
        for (int q = threadIdx.x; q < Ttok * k; q += blockDim.x) {
            const int id = ids_out[q], tl = q / k;
            atomicOr(&bits[id * kWords + (tl >> 5)], 1u << (tl & 31));
            if (tl == me) my_ids[q - tl * k] = id;
        }
    }
    for (int tl = grp; tl < (picked ? 0 : Ttok); tl += ngrp) {   // whole lane groups iterate together
        {
            int id;
            float w;
            route_token(scores + static_cast<int64_t>(tl) * E, E, k, G, vpl, lig, id, w);
            if (lig < k) {
                atomicOr(&bits[id * kWords + (tl >> 5)], 1u << (tl & 31));
                if (tl == me) {
                    my_ids[lig] = id;
                    weights[static_cast<int64_t>(me) * k + lig] = from_f32<T>(w);
                    if (ids_out) ids_out[static_cast<int64_t>(me) * k + lig] = id;
                }
            }
        }
    }
    __syncthreads();
    word_prefix(bits, wordpre, count, E);
    __syncthreads();
    if (threadIdx.x < kWave) scan_experts(count, E);   // exclusive scan over experts, in place
    __syncthreads();
    if (me == 0)
        for (int e = threadIdx.x; e <= E; e += blockDim.x) off[e] = count[e];
    if (threadIdx.x < k) {
        int e = my_ids[threadIdx.x];
        int64_t pos = count[e] + rank_in_chunk(bits, wordpre, e, me);
        my_inv[threadIdx.x] = pos;
        inv[static_cast<int64_t>(me) * k + threadIdx.x] = pos;
        if (row_token) row_token[pos] = me;
    }
    if (Xp == nullptr) return;              // routing only: the caller reads X through row_token
    __syncthreads();
    expand_row(X, Xp, static_cast<int64_t>(me), H, k, my_inv, vec);
}

// ---- index form, few tokens: router gate, top-k, softmax, offsets, inverse permutation and
// row_token in ONE launch of ONE block.  Without row copies (the gate/up GEMM reads X through
// row_token) nothing in MoeSelect needs more than one block, and the bookkeeping needs every
// token's picks, so a single block of sixteen waves does it all:
//   1. logits on the MFMA 16x16x32 units: the tokens form TT tiles of 16, the 16 / TT waves of a tile
//      split K (wave kw takes k-steps kw, kw + 16/TT, ...; four steps of loads in flight) and hold
//      all ET expert tiles; partial sums meet in LDS and are added in wave order, + bias, rounded
//      once to T (Linear.py:32) -- written to `scores` and kept in LDS;
//   2. top-k / softmax per token by lane groups on the rounded logits (moe_route.h), bit matrix;
//   3. word prefixes, scan over experts -> expert_offset;
//   4. rank of every (token, slot) -> invert_permutation, row_token.
// What bounds it is the one CU it runs on: a CU's load path moves 64 bytes per clock, so the logits
// of 32 tokens (X 256 KB + Wg) cost it 8 us where the router kernel spreads them over 32 CUs.
// Measured per call inside a HIP graph (router gate + MoeSelect, index form; separate kernels ->
// this kernel): 8 experts, H = 4096: T = 1 7.3 -> 7.1 us, T = 8 8.7 -> 8.4, T = 16 8.2 -> 9.6, T = 32
// 8.6 -> 15.5; 64 experts, H = 2048: T = 1 10.6 -> 13.8, T = 32 13.0 -> 32.6.  A dependent launch
// costs about 4 us there, less than one CU needs for the logits of a second tile of tokens, so the
// kernel is used up to kIndexOneLaunchTokens tokens and kIndexOneLaunchExperts experts and the
// separate kernels (each on as many CUs as it has tokens) beyond.
constexpr int kIndexWaves = 16;
constexpr int kIndexMaxTokens = 64;          // what the kernel can do (four token tiles)
template <typename T, int TT, int ET>
__global__ __launch_bounds__(kIndexWaves * 64) void route_index_kernel(const T *__restrict__ X, const T *__restrict__ Wg,
                                                                       const T *__restrict__ Bg, int Ttok, int64_t H,
                                                                       int E, int k, int G, T *__restrict__ scores_out,
                                                                       T *__restrict__ weights, int64_t *__restrict__ inv,
                                                                       int64_t *__restrict__ off,
                                                                       int32_t *__restrict__ row_token,
                                                                       int32_t *__restrict__ ids_out)
{
    using frag = typename Mfma<T>::frag;
    constexpr int NWK = kIndexWaves / TT;                    // waves that split K for one token tile
    constexpr int kE = 64;                                   // experts this kernel handles (one key per lane)
    extern __shared__ __attribute__((aligned(16))) char dyn[];
    float *part = reinterpret_cast<float *>(dyn);            // [kIndexWaves][ET][64][4]
    __shared__ T s_scores[kIndexMaxTokens * kE];
    __shared__ uint32_t bits[kE * kWords];
    __shared__ int wordpre[kE * kWords];
    __shared__ int count[kE + 1];
    __shared__ int s_ids[kIndexMaxTokens * OPMX_MOE_MAX_EXPERTS_PER_TOKEN];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int fr = lane & 15, fg = lane >> 4;
    {
        const int tt = wave % TT, kw = wave / TT;
        const int trow = tt * 16 + fr < Ttok ? tt * 16 + fr : Ttok - 1;      // padded token rows repeat the last one
        const T *xp = X + static_cast<int64_t>(trow) * H + fg * 8;
        const T *wp[ET];
#pragma unroll
        for (int e = 0; e < ET; ++e) {
            const int erow = e * 16 + fr < E ? e * 16 + fr : E - 1;            // padded expert rows likewise
            wp[e] = Wg + static_cast<int64_t>(erow) * H + fg * 8;
        }
        float4_t acc[ET];
#pragma unroll
        for (int e = 0; e < ET; ++e) acc[e] = float4_t{0.f, 0.f, 0.f, 0.f};
        const int steps = static_cast<int>(H / 32);
        int st = kw;
        // U k-steps of loads in flight at a time: the phase costs about one memory round trip per batch
#define OPMX_KBATCH(U)                                                                                     \
        for (; st + ((U)-1) * NWK < steps; st += (U)*NWK) {                                                \
            frag b[U], a[U][ET];                                                                           \
            _Pragma("unroll") for (int u = 0; u < (U); ++u) {                                              \
                b[u] = *reinterpret_cast<const frag *>(xp + (st + NWK * u) * 32);                          \
                _Pragma("unroll") for (int e = 0; e < ET; ++e)                                             \
                    a[u][e] = *reinterpret_cast<const frag *>(wp[e] + (st + NWK * u) * 32);                \
            }                                                                                              \
            _Pragma("unroll") for (int u = 0; u < (U); ++u)                                                \
                _Pragma("unroll") for (int e = 0; e < ET; ++e) acc[e] = Mfma<T>::m16(a[u][e], b[u], acc[e]); \
        }
        if constexpr (ET == 1) OPMX_KBATCH(8)
        OPMX_KBATCH(4)
        OPMX_KBATCH(2)
        OPMX_KBATCH(1)
#undef OPMX_KBATCH
        // acc[e][i]: expert e*16 + fg*4 + i, token tt*16 + fr
#pragma unroll
        for (int e = 0; e < ET; ++e) *reinterpret_cast<float4_t *>(part + ((wave * ET + e) * 64 + lane) * 4) = acc[e];
    }
    zero_bits(bits, E);
    __syncthreads();
    for (int q = threadIdx.x; q < Ttok * E; q += blockDim.x) {
        const int t = q / E, e = q - t * E;
        const int tt = t >> 4, idx = (((e >> 4) * 64) + (((e & 15) >> 2) * 16 + (t & 15))) * 4 + (e & 3);
        float v = 0.0f;
#pragma unroll
        for (int kw = 0; kw < NWK; ++kw) v += part[(kw * TT + tt) * ET * 64 * 4 + idx];
        if (Bg) v += to_f32(Bg[e]);
        const T r = from_f32<T>(v);
        s_scores[q] = r;
        scores_out[q] = r;
    }
    __syncthreads();
    const int lig = threadIdx.x % G, grp = threadIdx.x / G, ngrp = kIndexWaves * 64 / G;
    for (int tl = grp; tl < Ttok; tl += ngrp) {                 // whole lane groups iterate together
        int id;
        float w;
        route_token(s_scores + tl * E, E, k, G, 1, lig, id, w);
        if (lig < k) {
            atomicOr(&bits[id * kWords + (tl >> 5)], 1u << (tl & 31));
            s_ids[tl * k + lig] = id;
            weights[tl * k + lig] = from_f32<T>(w);
            if (ids_out) ids_out[tl * k + lig] = id;
        }
    }
    __syncthreads();
    word_prefix(bits, wordpre, count, E);
    __syncthreads();
    if (threadIdx.x < kWave) scan_experts(count, E);            // exclusive scan over experts, in place
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) off[e] = count[e];
    for (int q = threadIdx.x; q < Ttok * k; q += blockDim.x) {
        const int t = q / k, e = s_ids[q];
        const int pos = count[e] + rank_in_chunk(bits, wordpre, e, t);
        inv[q] = pos;
        row_token[pos] = t;
    }
}

// The buffer select_impl keeps the picked ids in: the caller's, or a part of the workspace.
inline int32_t *picks_buffer(int64_t Ttok, int E, int32_t *ids, void *ws)
{
    const int nchunks = static_cast<int>(ceil_div(Ttok, kChunk));
    return ids ? ids : reinterpret_cast<int32_t *>(static_cast<char *>(ws) + ceil_div(sizeof(int32_t) * nchunks * E, 256) * 256);
}

// scores_ == nullptr (more than kChunk tokens only): the picks are made -- expert ids in
// picks_buffer(), weights in w_ -- and the top-k kernel is skipped.
template <typename T>
int select_impl(const void *X_, const void *scores_, int64_t Ttok, int64_t H, int E, int k, void *Xp_, void *w_,
                int64_t *inv, int64_t *off, int32_t *ids, void *ws, hipStream_t s, int32_t *row_token)
{
    const T *X = static_cast<const T *>(X_);
    const T *scores = static_cast<const T *>(scores_);
    T *Xp = static_cast<T *>(Xp_);
    T *w = static_cast<T *>(w_);
    int G = 8;
    while (G < E && G < kWave) G <<= 1;
    const int vpl = (E + G - 1) / G;
    const bool vec = (H * sizeof(T)) % 16 == 0 && aligned16(X) && aligned16(Xp);
    const int64_t R = Ttok * k;

    if (Ttok == 0) {   // offsets are all zero; nothing else to write
        select_scan_kernel<<<1, 256, 0, s>>>(nullptr, 0, E, 0, off);
        OPMX_LAUNCH_CHECK();
        return OPMX_OK;
    }
    // Up to kChunk tokens.  One launch while routing every token in every block is cheap
    // (measured: 4.8 us at T = 32 with 8 experts, 7 us at T = 4 with 64; but 14 us at T = 32 with
    // 64 experts and 15 us at T = 256 with 8); beyond that the picks are made once per token by
    // select_topk_kernel and the same kernel does only the bookkeeping: 6-7 us for any such T.
    if (G == 8 ? Ttok <= 64 : (Ttok <= 16 && Ttok * G <= 512)) {
        // wide lane groups (many experts) route few tokens per wave: use a big block
        const unsigned threads = G >= 32 ? 1024 : kChunk;
        select_small_kernel<T, false><<<static_cast<unsigned>(Ttok), threads, 0, s>>>(
            X, scores, static_cast<int>(Ttok), H, E, k, G, vpl, Xp, w, inv, off, ids, vec, nullptr, nullptr, nullptr, row_token);
        OPMX_LAUNCH_CHECK();
        return OPMX_OK;
    }
    const int nchunks = static_cast<int>(ceil_div(Ttok, kChunk));
    char *wsb = static_cast<char *>(ws);
    int32_t *hist = reinterpret_cast<int32_t *>(wsb);
    int32_t *idbuf = picks_buffer(Ttok, E, ids, ws);
    if (Ttok <= kChunk) {
        select_topk_kernel<T><<<static_cast<unsigned>(ceil_div(Ttok, kChunk / G)), kChunk, 0, s>>>(scores, Ttok, E, k, G,
                                                                                                   vpl, w, idbuf);
        OPMX_LAUNCH_CHECK();
        select_small_kernel<T, false><<<static_cast<unsigned>(Ttok), kChunk, 0, s>>>(
            X, nullptr, static_cast<int>(Ttok), H, E, k, G, vpl, Xp, w, inv, off, idbuf, vec, nullptr, nullptr, nullptr, row_token);
        OPMX_LAUNCH_CHECK();
        return OPMX_OK;
    }
    if (scores != nullptr) {
        select_topk_kernel<T><<<static_cast<unsigned>(ceil_div(Ttok, kChunk / G)), kChunk, 0, s>>>(scores, Ttok, E, k, G,
                                                                                                   vpl, w, idbuf);
        OPMX_LAUNCH_CHECK();
    }
    select_hist_kernel<<<nchunks, kChunk, 0, s>>>(idbuf, Ttok, E, k, hist);
    OPMX_LAUNCH_CHECK();
    select_scan_kernel<<<1, E > 16 ? 1024 : 256, 0, s>>>(hist, nchunks, E, R, off);
    OPMX_LAUNCH_CHECK();
    select_rank_kernel<<<nchunks, kChunk, 0, s>>>(idbuf, hist, off, Ttok, E, k, inv, row_token);
    OPMX_LAUNCH_CHECK();
    if (Xp != nullptr) {                   // nullptr: routing only, the caller reads X through row_token
        const unsigned grid = static_cast<unsigned>(Ttok < 65536 ? Ttok : 65536);
        select_expand_kernel<T><<<grid, 256, 0, s>>>(X, Xp, inv, Ttok, H, k, vec);
        OPMX_LAUNCH_CHECK();
    }
    return OPMX_OK;
}

template <typename T>
int route_select_fused(const void *X_, const void *Wg_, const void *Bg_, int64_t Ttok, int64_t H, int E, int k,
                       void *scores_, void *Xp_, void *w_, int64_t *inv, int64_t *off, int32_t *ids, hipStream_t s,
                       int32_t *row_token)
{
    const T *X = static_cast<const T *>(X_);
    T *Xp = static_cast<T *>(Xp_);
    int G = 8;
    while (G < E) G <<= 1;
    const bool vec = (H * sizeof(T)) % 16 == 0 && aligned16(X) && aligned16(Xp);   // (unused without Xp)
    select_small_kernel<T, true><<<static_cast<unsigned>(Ttok), kFusedWaves * kWave, 0, s>>>(
        X, nullptr, static_cast<int>(Ttok), H, E, k, G, (E + G - 1) / G, Xp, static_cast<T *>(w_), inv, off, ids, vec,
        static_cast<const T *>(Wg_), static_cast<const T *>(Bg_), static_cast<T *>(scores_), row_token);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

// Up to how many tokens and experts route_index_kernel stands for the router kernel and the select
// kernels (measured against them on the Mixtral shape and with 64 experts, see the kernel).
constexpr int kIndexOneLaunchTokens = 8, kIndexOneLaunchExperts = 16;

template <typename T, int TT>
int route_index_launch(const T *X, const T *Wg, const T *Bg, int Ttok, int64_t H, int E, int k, T *scores, T *w,
                       int64_t *inv, int64_t *off, int32_t *row_token, int32_t *ids, hipStream_t s)
{
    int G = 8;
    while (G < E) G <<= 1;                       // E <= 64: one key per lane
    const int ET = (E + 15) / 16;
    static std::atomic<uint64_t> attr_done[3];
#define OPMX_ROUTE_INDEX(ETV, SLOT)                                                                         \
    do {                                                                                                    \
        auto kern = route_index_kernel<T, TT, ETV>;                                                         \
        constexpr int smem = kIndexWaves * ETV * 64 * 4 * static_cast<int>(sizeof(float));                  \
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done[SLOT])) return OPMX_ERR_LAUNCH; \
        kern<<<1, kIndexWaves * 64, smem, s>>>(X, Wg, Bg, Ttok, H, E, k, G, scores, w, inv, off, row_token, ids); \
    } while (0)
    if (ET == 1) OPMX_ROUTE_INDEX(1, 0);
    else if (ET == 2) OPMX_ROUTE_INDEX(2, 1);
    else OPMX_ROUTE_INDEX(4, 2);
#undef OPMX_ROUTE_INDEX
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T>
int route_index(const void *X, const void *Wg, const void *Bg, int64_t Ttok, int64_t H, int E, int k, void *scores,
                void *w, int64_t *inv, int64_t *off, int32_t *row_token, int32_t *ids, hipStream_t s)
{
    const T *x = static_cast<const T *>(X), *wg = static_cast<const T *>(Wg), *bg = static_cast<const T *>(Bg);
    T *sc = static_cast<T *>(scores), *wt = static_cast<T *>(w);
    const int t = static_cast<int>(Ttok);
    if (t <= 16) return route_index_launch<T, 1>(x, wg, bg, t, H, E, k, sc, wt, inv, off, row_token, ids, s);
    if (t <= 32) return route_index_launch<T, 2>(x, wg, bg, t, H, E, k, sc, wt, inv, off, row_token, ids, s);
    return route_index_launch<T, 4>(x, wg, bg, t, H, E, k, sc, wt, inv, off, row_token, ids, s);
}

}  // namespace

// Router gate and MoeSelect in one call.  One launch when the logits of all tokens fit one
// MFMA tile per block and that pays (fp16/bf16, T <= 8, E <= 16, H a multiple of 32, 16-byte aligned rows);
// otherwise the two operators one after the other.  `scores` [T,E] receives the logits either way.
int launch_moe_route_select(const void *X, const void *Wg, const void *Bg, int64_t T, int64_t H, int E, int k,
                            int dtype, void *scores, void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids,
                            void *ws, hipStream_t s, int32_t *row_token)
{
    const bool lowp = dtype == OPMX_DTYPE_F16 || dtype == OPMX_DTYPE_BF16;
    static_assert(kFusedMaxTokens <= kFusedTokens, "one MFMA tile of tokens");
    static_assert(kIndexOneLaunchTokens <= kIndexMaxTokens, "four token tiles");
    // Index form (no row copies), few tokens, up to 64 experts: everything in one launch of one block.
    // (the knob lifts both limits: up to 64 tokens and 64 experts, what the kernel can do)
    const bool knob = option(kOptRouteIndexTokens) >= 0;
    const int one_launch = knob ? option(kOptRouteIndexTokens) : kIndexOneLaunchTokens;
    if (lowp && Xp == nullptr && row_token != nullptr && T >= 1 && T <= one_launch && T <= kIndexMaxTokens &&
        E <= (knob ? 64 : kIndexOneLaunchExperts) &&
        H >= 32 && H % 32 == 0 && aligned16(X) && aligned16(Wg)) {
        if (dtype == OPMX_DTYPE_F16) return route_index<f16>(X, Wg, Bg, T, H, E, k, scores, w, inv, off, row_token, ids, s);
        return route_index<bf16>(X, Wg, Bg, T, H, E, k, scores, w, inv, off, row_token, ids, s);
    }
    if (lowp && T >= 1 && T <= kFusedMaxTokens && E <= kFusedExperts && H >= 32 && H % 32 == 0 && aligned16(X) &&
        aligned16(Wg)) {
        if (dtype == OPMX_DTYPE_F16)
            return route_select_fused<f16>(X, Wg, Bg, T, H, E, k, scores, Xp, w, inv, off, ids, s, row_token);
        return route_select_fused<bf16>(X, Wg, Bg, T, H, E, k, scores, Xp, w, inv, off, ids, s, row_token);
    }
    // Many tokens, few experts: the router kernel that holds a token's logits in one block routes
    // it as well, and MoeSelect starts from the picks (one launch and the read-back of the logits less).
    if (T > kChunk &&
        launch_linear_route(X, Wg, Bg, T, H, E, k, dtype, scores, w, picks_buffer(T, E, ids, ws), s) == OPMX_OK)
        return launch_moe_select(X, nullptr, T, H, E, k, dtype, Xp, w, inv, off, ids, ws, s, row_token);
    const int rc = launch_linear(X, Wg, Bg, T, H, E, dtype, scores, s);
    if (rc != OPMX_OK) return rc;
    return launch_moe_select(X, scores, T, H, E, k, dtype, Xp, w, inv, off, ids, ws, s, row_token);
}

size_t moe_select_workspace_bytes(int64_t T, int E, int k)
{
    if (T <= 0) return 256;
    const int64_t nchunks = ceil_div(T, kChunk);
    return static_cast<size_t>(ceil_div(sizeof(int32_t) * nchunks * E, 256) * 256 +
                               ceil_div(sizeof(int32_t) * T * k, 256) * 256);
}

int launch_moe_select(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                      void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids, void *ws, hipStream_t s,
                      int32_t *row_token)
{
    switch (dtype) {
        case OPMX_DTYPE_F32: return select_impl<float>(X, scores, T, H, E, k, Xp, w, inv, off, ids, ws, s, row_token);
        case OPMX_DTYPE_F16: return select_impl<f16>(X, scores, T, H, E, k, Xp, w, inv, off, ids, ws, s, row_token);
        case OPMX_DTYPE_BF16: return select_impl<bf16>(X, scores, T, H, E, k, Xp, w, inv, off, ids, ws, s, row_token);
    }
    return OPMX_ERR_UNSUPPORTED;
}

// ---- MoeSelect for callers that cannot allocate ----
// The chunk histograms and the picked ids of the many-token path live in this array instead of a
// caller's workspace.  Each GPU holds its own copy at its own address; host code never uses the
// array's name as an address, only the pointer hipGetSymbolAddress returned for that GPU.
static __device__ __align__(256) unsigned char scratch[OPMX_MOE_SELECT_STATIC_SCRATCH_BYTES];

namespace {
std::mutex scratch_mutex;
void *scratch_ptr[kMaxDevices];   // by device ordinal; written under scratch_mutex

// The address of `scratch` on the GPU that is current on this thread (looked up once per GPU).
int scratch_for_current_device(void **out)
{
    const int dev = current_device();
    if (dev < 0) return OPMX_ERR_LAUNCH;
    std::lock_guard<std::mutex> hold(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return OPMX_ERR_LAUNCH;
        }
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return OPMX_OK;
}
}  // namespace

// Every kernel of select_impl writes the part of the scratch memory it later reads (all chunk
// histograms of the call, all picked ids), so nothing has to start at zero and what the
// previous call left behind is never read.
int launch_moe_select_static(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                             void *Xp, void *w, int64_t *inv, int64_t *off, int32_t *ids, hipStream_t s)
{
    if (moe_select_workspace_bytes(T, E, k) > sizeof(scratch)) return OPMX_ERR_WORKSPACE;
    void *ws = nullptr;
    const int rc = scratch_for_current_device(&ws);
    if (rc != OPMX_OK) return rc;
    return launch_moe_select(X, scores, T, H, E, k, dtype, Xp, w, inv, off, ids, ws, s, nullptr);
}

}  // namespace opmx
