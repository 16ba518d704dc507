// Grouped expert GEMM for gfx950, HBM-bound regime (few rows per expert: decode).
//
// The job is to read every active expert's W[e] [N,K] exactly once at HBM speed;
// the flops ride along on v_mfma_f32_16x16x32 with W as the A operand (16 weight
// rows per wave) and the expert's few X rows as the B operand.
//
//  * a block = 4 waves = 64 consecutive rows of W[e] (one 16-row group per wave; two groups,
//    128 rows per block, once the row tile is 64 rows or taller)
//    x one row tile (<= 16*MT rows) of expert e, over the whole K;
//  * W is fetched with fully coalesced 16-byte loads (a wave instruction reads
//    1 KiB contiguous) into registers, DEPTH K-chunks ahead, then transposed
//    into the MFMA operand layout through a wave-private LDS strip (no block
//    barrier for W);
//  * the X chunk is shared by the four waves through double-buffered LDS: one
//    barrier per K-chunk;
//  * experts with no rows produce no work, so their weights are never touched;
//  * optional SwiGLU epilogue: a wave streams 16 gate rows and the 16 matching up rows
//    (N/2 apart in W[e]) and combines the two accumulators in registers; or, for long K, a
//    pair of waves streams one of the two each and combines through LDS after the K loop.
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67 and
// torch_function/MoeRowParallelLinear.py:47-53 of OpenPPL/ppl.pmx.
#include "moe_gemm.h"

namespace opmx {
namespace {

// A block has SW waves (4 normally; 1 when the launch would otherwise leave CUs idle)
// and owns 16*SW consecutive rows of W[e].

template <bool NT> __device__ __forceinline__ u32x4 ld16(const char *p)
{
    if (NT) return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return *reinterpret_cast<const u32x4 *>(p);
}

// XR: X rows a tile holds and the block stages per K chunk.  16*MT normally; 2 for calls with at most two rows
// in all (a single token with two experts): the MFMA still multiplies 16 columns, the lanes of the
// fourteen that do not exist read the last staged row again, and the X chunk is 1 KiB instead of 8 --
// with one row per expert the sixteen-row staging moved as many bytes through LDS as the weights.
template <typename T, int MT, int KC, int DEPTH, bool NT, int SW, bool SG, bool PAIR, bool SGW = false, int XR = 16 * MT>
__global__ __launch_bounds__(SW * 64) void gemm_stream_kernel(const T *__restrict__ X,
                                                               const int64_t *__restrict__ off,
                                                               const T *__restrict__ W,
                                                               const T *__restrict__ Bias, int E, int64_t R,
                                                               int64_t K, int64_t N, T *__restrict__ Y,
                                                               const int32_t *__restrict__ rt, int64_t xrows)
{
    // row groups per wave: SwiGLU pairs gate rows with up rows; PAIR gives a wave two adjacent
    // groups, so that a block shares its X chunk among twice the weight rows (tall row tiles,
    // where the X chunk is as large as the weight chunk)
    // SGW: SwiGLU by wave pairs -- even waves stream gate rows, odd waves the matching up rows, one
    // group each (the LDS footprint and chunk width of the plain form), and the pair combines its
    // accumulators through LDS after the K loop.
    static_assert(!(SG && PAIR) && !(SGW && (SG || PAIR)) && (!SGW || SW % 2 == 0), "one or the other");
    constexpr int NG = (SG || PAIR) ? 2 : 1;
    constexpr int WROWS = PAIR ? 32 : 16;        // output columns per wave
    constexpr int SROWS = SGW ? 16 * SW / 2 : WROWS * SW;   // output columns per block
    constexpr int RS = KC * 2 + 16;              // LDS row stride in bytes (pad 16: conflict-free strips)
    constexpr int RPL = 512 / KC;                // W rows covered by one wave load (1 KiB)
    constexpr int NLW = 16 / RPL;                // W loads per wave per chunk
    constexpr int XM = XR;                       // X rows per tile
    constexpr int CPR = KC / 8;                  // 16-byte chunks per row per K-chunk
    constexpr bool XW0 = XM * CPR == 64 && SW > 1;                   // the X chunk is one wave load: every wave makes it
    constexpr int NLX = XW0 ? 1 : XM * CPR / (SW * 64);              // X loads per thread per chunk
    constexpr int WSTRIP = NG * 16 * RS;
    constexpr int XBUF = XM * RS;
    static_assert(XW0 || XM * CPR % (SW * 64) == 0, "X chunk must divide over the block");
    static_assert(XR == 16 * MT || (MT == 1 && XR < 16), "short tiles: one MFMA tile of rows");
    static_assert(DEPTH == 1 || DEPTH == 2, "one or two chunks in flight");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];   // [SW][WSTRIP] | [2][XBUF]

    const int64_t ND = (SG || SGW) ? N / 2 : N;  // output columns; with SwiGLU W rows n and ND+n pair up
    zero_unowned_rows(Y, R, ND, off, E);
    const MTile mt = find_mtile(off, E, R, XM, blockIdx.y);
    if (mt.rows == 0) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    char *wstrip = smem + wave * WSTRIP;
    char *xbuf = smem + SW * WSTRIP;

    // ---- this wave's 16 rows of W[e]: uniform base + per-lane byte offsets.
    // Rows past N are clamped to row N-1 (their results are masked at the store).
    const int64_t nbase = static_cast<int64_t>(blockIdx.x) * SROWS + (SGW ? (wave >> 1) * 16 : wave * WROWS);
    const char *wb = reinterpret_cast<const char *>(W + static_cast<int64_t>(mt.e) * N * K);
    // X rows of this tile: in place from row0 on, or through the row index (RowGather; x_rows * K * 2 < 2^32)
    const char *xb = reinterpret_cast<const char *>(rt ? X : X + mt.row0 * K);
    const int wl_row = lane / (64 / RPL);               // row inside one wave load
    const int wl_k = (lane % (64 / RPL)) * 8;           // k offset inside the chunk
    uint32_t wrow[NG][NLW];                             // byte offset of the row start
    int wdst[NG][NLW];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int i = 0; i < NLW; ++i) {
            const int row = i * RPL + wl_row;
            int64_t n = nbase + row + (PAIR ? g * 16 : 0);
            n = (n < ND ? n : ND - 1) + (SG ? g * ND : 0) + (SGW && (wave & 1) ? ND : 0);
            wrow[g][i] = static_cast<uint32_t>(n * K * 2);
            wdst[g][i] = (g * 16 + row) * RS + wl_k * 2;
        }
    uint32_t xrow[NLX];
    int xdst[NLX], xk[NLX];
#pragma unroll
    for (int i = 0; i < NLX; ++i) {
        // XW0: all waves load and stage the same 1 KiB (identical bytes to identical places: a branch that
        // left it to one wave would cost the others their load pipelining, the compiler then waits for everything)
        const int q = XW0 ? lane : tid + SW * 64 * i, row = q / CPR, c = q % CPR;
        const int r = row < mt.rows ? row : mt.rows - 1;
        xrow[i] = static_cast<uint32_t>((rt ? gathered_row(rt, xrows, mt.row0 + r) : r) * K * 2);
        xdst[i] = row * RS + c * 16;
        xk[i] = c * 8;
    }

    float4_t acc[NG][MT];
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[g][m] = float4_t{0.f, 0.f, 0.f, 0.f};

    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    u32x4 wreg[DEPTH][NG][NLW], xreg[DEPTH][NLX];
    const int nchunks = static_cast<int>((K + KC - 1) / KC);
    const int nfull = static_cast<int>(K / KC);          // chunks entirely inside K
    // Every block starts its walk over K at a different chunk (and wraps around).  Blocks that all
    // walk K from 0 advance in near lockstep, so at any moment all their loads sit at the same
    // offset inside rows that lie a power of two apart (K = 4096: 8 KiB) and crowd onto a few
    // memory channels: 5.95 TB/s for the Mixtral gate/up shape against 6.95 TB/s with the walks
    // spread out (K = 8192: 6.2 -> 6.8, K = 14336: 6.5 -> 6.7; with 8 chunks or fewer it does not
    // pay).  The order of the fp32 accumulation then differs from block to block, but is fixed.
    const int rot = nchunks >= 16 ? static_cast<int>((blockIdx.x * 7u + blockIdx.y * 3u) % static_cast<unsigned>(nchunks)) : 0;

#define OPMX_FETCH(SET, KCI)                                                                           \
    do {                                                                                               \
        const int seq_ = (KCI);                                                                        \
        const int kci_ = seq_ >= nchunks ? nchunks : (seq_ + rot >= nchunks ? seq_ + rot - nchunks : seq_ + rot); \
        if (kci_ < nfull) {                                                                            \
            const char *wk_ = wb + static_cast<int64_t>(kci_) * (KC * 2);                              \
            const char *xk_ = xb + static_cast<int64_t>(kci_) * (KC * 2);                              \
            _Pragma("unroll") for (int g = 0; g < NG; ++g)                                             \
                _Pragma("unroll") for (int i = 0; i < NLW; ++i)                                        \
                    wreg[SET][g][i] = ld16<NT>(wk_ + (wrow[g][i] + static_cast<uint32_t>(wl_k * 2)));  \
            _Pragma("unroll") for (int i = 0; i < NLX; ++i)                                            \
                xreg[SET][i] = ld16<false>(xk_ + (xrow[i] + static_cast<uint32_t>(xk[i] * 2)));        \
        } else if (kci_ < nchunks) { /* ragged last chunk: lanes past K read the row start, get 0 */   \
            const int64_t k0_ = static_cast<int64_t>(kci_) * KC;                                       \
            _Pragma("unroll") for (int g = 0; g < NG; ++g)                                             \
                _Pragma("unroll") for (int i = 0; i < NLW; ++i) {                                      \
                    const bool in_ = k0_ + wl_k < K;                                                   \
                    const u32x4 v_ = ld16<false>(wb + (wrow[g][i] + (in_ ? static_cast<uint32_t>((k0_ + wl_k) * 2) : 0u))); \
                    wreg[SET][g][i] = in_ ? v_ : zero4;                                                \
                }                                                                                      \
            _Pragma("unroll") for (int i = 0; i < NLX; ++i) {                                          \
                const bool in_ = k0_ + xk[i] < K;                                                      \
                const u32x4 v_ = ld16<false>(xb + (xrow[i] + (in_ ? static_cast<uint32_t>((k0_ + xk[i]) * 2) : 0u))); \
                xreg[SET][i] = in_ ? v_ : zero4;                                                       \
            }                                                                                          \
        }                                                                                              \
    } while (0)

    const int fr = lane & 15, fg = lane >> 4;   // fragment row (W row / X row) and k group
    const int xfr = XR >= 16 ? fr : (fr < XR ? fr : XR - 1);   // ... the staged X row this lane reads

#define OPMX_STEP(SET, KCI)                                                                            \
    do {                                                                                               \
        char *xcur_ = xbuf + ((KCI)&1) * XBUF;                                                         \
        _Pragma("unroll") for (int g = 0; g < NG; ++g)                                                 \
            _Pragma("unroll") for (int i = 0; i < NLW; ++i)                                            \
                *reinterpret_cast<u32x4 *>(wstrip + wdst[g][i]) = wreg[SET][g][i];                     \
        _Pragma("unroll") for (int i = 0; i < NLX; ++i)                                                \
            *reinterpret_cast<u32x4 *>(xcur_ + xdst[i]) = xreg[SET][i];                                \
        OPMX_FETCH(SET, (KCI) + DEPTH);                                                                \
        __syncthreads();                                                                               \
        _Pragma("unroll") for (int s = 0; s < KC / 32; ++s) {                                          \
            const int c_ = s * 4 + fg;                                                                 \
            frag a_[NG];                                                                               \
            _Pragma("unroll") for (int g = 0; g < NG; ++g)                                             \
                a_[g] = *reinterpret_cast<const frag *>(wstrip + (g * 16 + fr) * RS + c_ * 16);        \
            _Pragma("unroll") for (int m = 0; m < MT; ++m) {                                           \
                const frag b_ = *reinterpret_cast<const frag *>(xcur_ + (m * 16 + xfr) * RS + c_ * 16); \
                _Pragma("unroll") for (int g = 0; g < NG; ++g)                                         \
                    acc[g][m] = Mfma<T>::m16(a_[g], b_, acc[g][m]);                                    \
            }                                                                                          \
        }                                                                                              \
    } while (0)

    OPMX_FETCH(0, 0);
    if (DEPTH == 2) OPMX_FETCH(DEPTH - 1, 1);
    if (DEPTH == 1) {
        for (int kc = 0; kc < nchunks; ++kc) OPMX_STEP(0, kc);
    } else {
        int kc = 0;
        for (; kc + 1 < nchunks; kc += 2) {
            OPMX_STEP(0, kc);
            OPMX_STEP(DEPTH - 1, kc + 1);
        }
        if (kc < nchunks) OPMX_STEP(0, kc);
    }
#undef OPMX_STEP
#undef OPMX_FETCH

    float4_t up[MT];                 // SGW: the partner wave's accumulators (the up projection)
    if constexpr (SGW) {
        __syncthreads();             // every wave is done with the staging memory
        float *exch = reinterpret_cast<float *>(smem);   // [SW/2][MT][64 lanes][4]
        if (wave & 1) {
#pragma unroll
            for (int m = 0; m < MT; ++m)
                *reinterpret_cast<float4_t *>(exch + (((wave >> 1) * MT + m) * 64 + lane) * 4) = acc[0][m];
        }
        __syncthreads();
        if (wave & 1) return;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            up[m] = *reinterpret_cast<const float4_t *>(exch + (((wave >> 1) * MT + m) * 64 + lane) * 4);
    }
    // acc[g][m][i]: output column nbase + fg*4 + i (W row g*ND + that), X row m*16 + fr
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int row = m * 16 + fr;
        if (row >= mt.rows) continue;
        T *yrow = Y + (mt.row0 + row) * ND;
#pragma unroll
        for (int g = 0; g < (PAIR ? 2 : 1); ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t n = nbase + g * 16 + fg * 4 + i;
                if (n >= ND) continue;
                float v = acc[g][m][i];
                if (Bias) v += to_f32(Bias[static_cast<int64_t>(mt.e) * N + n]);
                if (SG || SGW) {                   // SwiGLU.py:15-16 on the fp32 accumulators, beta = 1
                    float u = SGW ? up[m][i] : acc[NG - 1][m][i];
                    if (Bias) u += to_f32(Bias[static_cast<int64_t>(mt.e) * N + ND + n]);
                    v = u * v * sigmoid_fast_(v);
                }
                yrow[n] = from_f32<T>(v);
            }
    }
}

template <typename T, int MT, int KC, int DEPTH, bool NT, int SW, bool SG, bool PAIR = false, bool SGW = false, int XR = 16 * MT>
int stream_launch_sw(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                     int64_t N, void *Y, hipStream_t s, RowGather g)
{
    constexpr int SROWS = SGW ? 16 * SW / 2 : (PAIR ? 32 : 16) * SW;
    constexpr int RS = KC * 2 + 16;
    constexpr int smem = SW * ((SG || PAIR) ? 2 : 1) * 16 * RS + 2 * XR * RS;
    static_assert(!SGW || (SW / 2) * MT * 1024 <= smem, "the pair exchange reuses the staging memory");
    auto kern = gemm_stream_kernel<T, MT, KC, DEPTH, NT, SW, SG, PAIR, SGW, XR>;
    static std::atomic<uint64_t> attr_done{0};
    if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done)) return OPMX_ERR_LAUNCH;
    dim3 grid(static_cast<unsigned>(ceil_div((SG || SGW) ? N / 2 : N, SROWS)),
              static_cast<unsigned>(max_mtiles(R, E, XR)));
    kern<<<grid, SW * 64, smem, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                     static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), g.index, g.x_rows);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T, int MT, int KC, int DEPTH, bool NT, bool SG = false>
int stream_launch(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                  int64_t N, void *Y, hipStream_t s, RowGather g)
{
    // at most min(R, E) experts are active: with 64-column blocks that is this many work items
    const int64_t items = ceil_div(SG ? N / 2 : N, 64) * (R < E ? R : E);
    if (MT <= 2 && items < 512)
        return stream_launch_sw<T, MT, KC, DEPTH, NT, 1, SG>(X, off, W, B, E, R, K, N, Y, s, g);
    // Tall row tiles: the X chunk a block stages is as large as its weight chunk, so every wave takes
    // two groups of weight rows and the block shares X among 128 of them (Mixtral gate/up at
    // T = 128: 357 -> 337 us, 64-row tiles; T = 256, 128-row tiles: 497 -> 374 us).
    if constexpr (MT >= 4 && !SG)
        return stream_launch_sw<T, MT, KC, DEPTH, NT, 4, SG, true>(X, off, W, B, E, R, K, N, Y, s, g);
    return stream_launch_sw<T, MT, KC, DEPTH, NT, 4, SG>(X, off, W, B, E, R, K, N, Y, s, g);
}

// Row-tile height MT*16 from the rows-per-expert bound m; K-chunk width per height
// (narrower chunks for taller tiles keep the LDS footprint, hence occupancy, level).
template <typename T, int KC1, int KC2, int KC4, int KC8, int DEPTH, bool NT>
int stream_pick_mt(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                   int64_t N, int64_t m, void *Y, hipStream_t s, RowGather g)
{
    // A short K (fewer than 16 chunks of 256) is walked in chunks of 128: a block then lives for a
    // few chunks only, and the narrower chunks halve its LDS footprint, so that twice as many
    // blocks per CU overlap each other's start and end (64 experts, H = 2048, I = 1408, bf16:
    // layer at T = 32 0.255 -> 0.211 ms, at T = 1 0.189 -> 0.126 ms).
    constexpr int KC1S = KC1 > 128 ? 128 : KC1, KC2S = KC2 > 128 ? 128 : KC2, KC4S = KC4 > 64 ? 64 : KC4;
    const bool short_k = K < 16 * 256;
    // Up to 8 rows per expert (twice the mean, or the caller's bound): 16-row tiles.  The X chunk a block
    // stages is then half as large, which shows where blocks are single waves (few weight rows: the
    // Mixtral down projection at T = 8 ... 12, 131 -> 126 us); no difference at T = 16 or with 64 experts.
    if (m <= 8) {
        // at most two rows in all (one token, two experts): two-row X tiles, see the kernel's XR
        if constexpr (KC1 == 256 && DEPTH == 2 && NT)
            if (R <= 2 && !short_k) {
                if (ceil_div(N, 64) * R < 512)
                    return stream_launch_sw<T, 1, 256, 2, true, 1, false, false, false, 2>(X, off, W, B, E, R, K, N, Y, s, g);
                return stream_launch_sw<T, 1, 256, 2, true, 4, false, false, false, 2>(X, off, W, B, E, R, K, N, Y, s, g);
            }
        return short_k ? stream_launch<T, 1, KC1S, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g)
                       : stream_launch<T, 1, KC1, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g);
    }
    if (m <= 32)
        return short_k ? stream_launch<T, 2, KC2S, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g)
                       : stream_launch<T, 2, KC2, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g);
    // 64-row tiles: 64-wide chunks up to K = 8192 (Mixtral gate/up, K = 4096, at T = 128: 337 -> 322 us),
    // 128-wide beyond (down projection, K = 14336: 162 us against 175 with 64-wide chunks)
    if (m <= 64)
        return K <= 8192 ? stream_launch<T, 4, KC4S, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g)
                         : stream_launch<T, 4, KC4, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g);
    return stream_launch<T, 8, KC8, DEPTH, NT>(X, off, W, B, E, R, K, N, Y, s, g);
}

// SwiGLU epilogue: a wave streams twice the rows, so the K chunks are half as wide.
template <typename T>
int stream_swiglu_impl(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                       int64_t N, int64_t rows_hint, void *Y, hipStream_t s, RowGather g)
{
    const int64_t m = rows_hint > 0 ? rows_hint : R;
    if (m <= 2) {    // short K: narrower chunks, as in stream_pick_mt
        if (K >= 16 * 256 && ceil_div(N / 2, 64) * (R < E ? R : E) >= 256) {
            if (R <= 2)   // two-row X tiles, see the kernel's XR
                return stream_launch_sw<T, 1, 256, 2, true, 4, false, false, true, 2>(X, off, W, B, E, R, K, N, Y, s, g);
            return stream_launch_sw<T, 1, 256, 2, true, 4, false, false, true>(X, off, W, B, E, R, K, N, Y, s, g);
        }
        return K < 16 * 256 ? stream_launch<T, 1, 128, 2, true, true>(X, off, W, B, E, R, K, N, Y, s, g)
                            : stream_launch<T, 1, 256, 2, true, true>(X, off, W, B, E, R, K, N, Y, s, g);
    }
    if (m <= 32) {
        // long K: SwiGLU by wave pairs, which keeps the plain form's 256-wide chunks and LDS footprint
        // (a wave with two row groups needs twice the strip: chunks half as wide, or half the waves
        // per CU).  Decode T=32, layer: 0.452 ms with two groups per wave, 0.442 by pairs (unfused 0.440).
        const int64_t items = ceil_div(N / 2, 64) * (R < E ? R : E);
        if (K >= 16 * 256 && items >= 512)
            return stream_launch_sw<T, 2, 256, 2, true, 4, false, false, true>(X, off, W, B, E, R, K, N, Y, s, g);
        return stream_launch<T, 2, 128, 2, true, true>(X, off, W, B, E, R, K, N, Y, s, g);
    }
    if (m <= 64) return stream_launch<T, 4, 64, 2, true, true>(X, off, W, B, E, R, K, N, Y, s, g);
    return stream_launch<T, 8, 64, 2, true, true>(X, off, W, B, E, R, K, N, Y, s, g);
}

template <typename T>
int stream_impl(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                int64_t N, int64_t rows_hint, int variant, void *Y, hipStream_t s, RowGather g)
{
    const int64_t m = rows_hint > 0 ? rows_hint : R;
    switch (variant) {   // tuning knob; every variant computes the same thing
        case 1: return stream_pick_mt<T, 256, 256, 128, 128, 1, false>(X, off, W, B, E, R, K, N, m, Y, s, g);
        case 2: return stream_pick_mt<T, 512, 512, 256, 128, 1, true>(X, off, W, B, E, R, K, N, m, Y, s, g);
        case 3: return stream_pick_mt<T, 256, 256, 128, 64, 2, false>(X, off, W, B, E, R, K, N, m, Y, s, g);
        case 4: return stream_pick_mt<T, 256, 128, 64, 64, 2, true>(X, off, W, B, E, R, K, N, m, Y, s, g);
        case 5: return stream_pick_mt<T, 256, 256, 128, 128, 2, true>(X, off, W, B, E, R, K, N, m, Y, s, g);
        default: return stream_pick_mt<T, 256, 256, 128, 64, 2, true>(X, off, W, B, E, R, K, N, m, Y, s, g);
    }
}

}  // namespace

// Requires: dtype f16/bf16, K % 8 == 0, 16-byte aligned X and W.
int launch_gemm_stream(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                       int64_t K, int64_t N, int dtype, int epilogue, int64_t rows_hint, int variant, void *Y,
                       hipStream_t s, RowGather g)
{
    if (epilogue == OPMX_EPILOGUE_SWIGLU) {
        if (dtype == OPMX_DTYPE_F16) return stream_swiglu_impl<f16>(X, off, W, B, E, R, K, N, rows_hint, Y, s, g);
        if (dtype == OPMX_DTYPE_BF16) return stream_swiglu_impl<bf16>(X, off, W, B, E, R, K, N, rows_hint, Y, s, g);
        return OPMX_ERR_UNSUPPORTED;
    }
    switch (dtype) {
        case OPMX_DTYPE_F16: return stream_impl<f16>(X, off, W, B, E, R, K, N, rows_hint, variant, Y, s, g);
        case OPMX_DTYPE_BF16: return stream_impl<bf16>(X, off, W, B, E, R, K, N, rows_hint, variant, Y, s, g);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
