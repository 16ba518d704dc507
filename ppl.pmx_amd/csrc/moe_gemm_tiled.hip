// Grouped expert GEMM for gfx950, MFMA-bound regime (many rows per expert).
//
//   Y[r, :] = X[r, :] W[e]^T (+ B[e])   for off[e] <= r < off[e+1]
//
// X [R,K] and W[e] [N,K] are both K-contiguous, so A and B fragments of
// v_mfma_f32_32x32x16_{f16,bf16} are 16-byte loads.  A block owns a BM x BN
// output tile of ONE expert (tiles never straddle experts; the tile list is
// derived on the device from expert_offset, no host sync), stages X and W
// tiles of BK=64 through XOR-swizzled LDS (two LDS buffers, one barrier per
// k-tile, loads and LDS stores software-pipelined between the MFMA groups; with
// ILV the instruction order inside a group is pinned to MFMA / fragment read /
// LDS store / global load round-robin so the matrix pipe never waits behind a
// burst of memory instructions) and accumulates in fp32.  Optional SwiGLU
// epilogue on the accumulators (gate rows i and up rows N/2+i of W are placed
// in the same lane by the B-tile row order).
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67,
// torch_function/MoeRowParallelLinear.py:47-53, torch_function/SwiGLU.py:15-16.
#include <cstdlib>

#include "moe_gemm.h"

namespace opmx {
namespace {

constexpr int BK = 64;                 // k elements per LDS tile (128 bytes per row)
constexpr int ROWB = BK * 2;           // bytes per LDS row
constexpr int CH = ROWB / 16;          // 16-byte chunks per row (8)

// Byte offset of 16-byte chunk `chunk` of tile row `row`.  Rows are 128 bytes; the
// XOR with (row>>1)&7 spreads 16 consecutive rows of one chunk column over all
// sixteen 16-byte bank groups of a 256-byte LDS line pair (conflict-free b128 reads).
__device__ __forceinline__ int lds_off(int row, int chunk) { return row * ROWB + ((chunk ^ ((row >> 1) & 7)) << 4); }

template <typename T, int BM, int BN, int WM, int WN, bool SWIGLU, bool ILV>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tiled_kernel(const T *__restrict__ X,
                                                                  const int64_t *__restrict__ off,
                                                                  const T *__restrict__ W,
                                                                  const T *__restrict__ Bias, int E, int64_t R,
                                                                  int64_t K, int64_t N, T *__restrict__ Y,
                                                                  int ntiles_m, int ntiles_n, int gnx)
{
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    constexpr int BNO = SWIGLU ? BN / 2 : BN;            // output columns per tile
    constexpr int LA = BM * CH / NT, LB = BN * CH / NT;  // 16-byte loads per thread per k-tile
    constexpr int STAGE = (BM + BN) * ROWB;
    static_assert(BM * CH % NT == 0 && BN * CH % NT == 0, "tile/threads mismatch");
    static_assert(!SWIGLU || TN % 2 == 0, "SwiGLU needs an even number of n sub-tiles per wave");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int64_t s_off[OPMX_MOE_MAX_EXPERTS + 1];

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);

    // Block -> tile map.  Workgroups are handed to the 8 XCDs round-robin by linear id and
    // each XCD has its own L2, so 256 consecutive ids ("a round": 32 per XCD) are laid out
    // as a gm x (8*gnx) block of tiles in which XCD j owns a compact gm x gnx sub-block:
    // its 32 resident blocks share gm X-tiles and gnx W-tiles in L2, and all 8 XCDs share
    // the round's X-tiles through the memory-side cache.  Rounds walk n first, then m.
    int tile_m, tile_n;
    if (gnx > 0) {
        const int gm = 32 / gnx;
        const int lin = blockIdx.x, xcd = lin & 7, slot = (lin >> 3) & 31, round = lin >> 8;
        const int rounds_n = (ntiles_n + 8 * gnx - 1) / (8 * gnx);
        tile_m = (round / rounds_n) * gm + slot % gm;
        tile_n = (round % rounds_n) * (8 * gnx) + xcd * gnx + slot / gm;
    } else {                       // plain row-major order, n fastest
        tile_m = blockIdx.x / ntiles_n;
        tile_n = blockIdx.x % ntiles_n;
    }
    if (tile_m >= ntiles_m || tile_n >= ntiles_n) return;
    const MTile mt = find_mtile(off, E, R, BM, tile_m, s_off);
    if (mt.rows == 0) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int64_t n0 = static_cast<int64_t>(tile_n) * BNO;
    const T *Xt = X + mt.row0 * K;
    const T *We = W + static_cast<int64_t>(mt.e) * N * K;

    // per-thread global offsets (elements) and LDS offsets (bytes) of its loads
    int a_src[LA], a_dst[LA], b_src[LB], b_dst[LB];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int q = tid + NT * i, row = q / CH, c = q % CH;
        const int r = row < mt.rows ? row : mt.rows - 1;
        a_src[i] = static_cast<int>(r * K + c * 8);
        a_dst[i] = lds_off(row, c);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int q = tid + NT * i, row = q / CH, c = q % CH;
        int64_t wrow;
        if (SWIGLU) {
            const int w = row / WTN, jj = row % WTN, half = jj / (WTN / 2);
            int64_t ii = n0 + w * (WTN / 2) + jj % (WTN / 2);
            ii = ii < ncols ? ii : ncols - 1;
            wrow = half * ncols + ii;
        } else {
            wrow = n0 + row < N ? n0 + row : N - 1;
        }
        b_src[i] = static_cast<int>(wrow * K + c * 8);
        b_dst[i] = BM * ROWB + lds_off(row, c);
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // Software pipeline over k-tiles: ONE register set for global->LDS staging, two LDS
    // buffers, double-buffered MFMA fragments, one barrier per k-tile.
    // An iteration (tile kt in LDS buffer kt&1) has KS = BK/16 MFMA groups.  Group g
    //   - prefetches the fragments of group g+1 into the other fragment set,
    //   - issues its MFMAs on fragments that were fetched one group earlier,
    //   - (g < KS-1) stores its share of the staging registers (tile kt+1, loaded one
    //     iteration ago) into LDS buffer (kt+1)&1 and reloads them with tile kt+2.
    // The barrier sits BEFORE the last group: by then every wave has finished reading
    // buffer kt&1 (the last group's fragments are already in registers) and writing
    // buffer (kt+1)&1, so the last group prefetches the first fragments of tile kt+1
    // while its MFMAs run, and the next iteration may overwrite buffer kt&1.
    constexpr int KS = BK / 16, NQ = LA + LB, QPK = (NQ + KS - 2) / (KS - 1);
    // first MFMA slot that carries an LDS-store/global-load pair: LDS stores stay behind the group's fragment reads
    constexpr int ILV0 = TM + TN < TM * TN - QPK ? TM + TN : (TM * TN - QPK > 0 ? TM * TN - QPK : 0);
    u32x4 rq[NQ];
    frag fa[2][TM], fb[2][TN];
    const int nk = static_cast<int>(K / BK);
    const int lrow = lane & 31, lk = lane >> 5;
    int fa_off[TM], fb_off[TN];      // LDS offsets of this lane's fragments for chunk pair 0
#pragma unroll
    for (int i = 0; i < TM; ++i) fa_off[i] = (wm * WTM + i * 32 + lrow) * ROWB;
#pragma unroll
    for (int j = 0; j < TN; ++j) fb_off[j] = BM * ROWB + (wn * WTN + j * 32 + lrow) * ROWB;
    const int swz = (lrow >> 1) & 7;  // (row>>1)&7 of every fragment row of this lane (rows differ by multiples of 32)

#define OPMX_LOADQ(Q, KT)                                                                          \
    do {                                                                                           \
        const int64_t ko_ = static_cast<int64_t>(KT) * BK;                                         \
        if ((Q) < LA) rq[Q] = *reinterpret_cast<const u32x4 *>(Xt + a_src[(Q) < LA ? (Q) : 0] + ko_); \
        else rq[Q] = *reinterpret_cast<const u32x4 *>(We + b_src[(Q) < LA ? 0 : (Q)-LA] + ko_);    \
    } while (0)
#define OPMX_DRAINQ(Q, BUF)                                                                        \
    do {                                                                                           \
        char *dst_ = smem + (BUF)*STAGE;                                                           \
        if ((Q) < LA) *reinterpret_cast<u32x4 *>(dst_ + a_dst[(Q) < LA ? (Q) : 0]) = rq[Q];        \
        else *reinterpret_cast<u32x4 *>(dst_ + b_dst[(Q) < LA ? 0 : (Q)-LA]) = rq[Q];              \
    } while (0)
#define OPMX_FRAGS(SET, BUF, G)                                                                    \
    do {                                                                                           \
        const char *src_ = smem + (BUF)*STAGE;                                                     \
        const int co_ = ((((G)*2 + lk) ^ swz) << 4);                                               \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                             \
            fa[SET][i] = *reinterpret_cast<const frag *>(src_ + fa_off[i] + co_);                  \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                             \
            fb[SET][j] = *reinterpret_cast<const frag *>(src_ + fb_off[j] + co_);                  \
    } while (0)
#define OPMX_MMA(SET)                                                                              \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                             \
            _Pragma("unroll") for (int j = 0; j < TN; ++j)                                         \
                acc[i][j] = Mfma<T>::m32(fa[SET][i], fb[SET][j], acc[i][j]);                       \
    } while (0)
#define OPMX_ITER(KT, DRAIN, LOAD, NEXT)                                                           \
    do {                                                                                           \
        _Pragma("unroll") for (int g = 0; g < KS - 1; ++g) {                                       \
            OPMX_FRAGS((g + 1) & 1, (KT)&1, g + 1);                                                \
            OPMX_MMA(g & 1);                                                                       \
            _Pragma("unroll") for (int qq = 0; qq < QPK; ++qq) {                                   \
                const int q = g * QPK + qq;                                                        \
                if (q < NQ) {                                                                      \
                    if (DRAIN) OPMX_DRAINQ(q, ((KT) + 1) & 1);                                     \
                    if (LOAD) OPMX_LOADQ(q, (KT) + 2);                                             \
                }                                                                                  \
            }                                                                                      \
            if (ILV) {                                                                             \
                _Pragma("unroll") for (int m = 0; m < TM * TN; ++m) {                              \
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                             \
                    if (m < TM + TN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);            \
                    if (m >= ILV0 && m < ILV0 + QPK && g * QPK + (m - ILV0) < NQ) {                \
                        if (DRAIN) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);              \
                        if (LOAD) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);               \
                    }                                                                              \
                }                                                                                  \
            }                                                                                      \
            __builtin_amdgcn_sched_barrier(0);                                                     \
        }                                                                                          \
        __syncthreads();                                                                           \
        if (NEXT) OPMX_FRAGS(KS & 1, ((KT) + 1) & 1, 0);                                           \
        OPMX_MMA((KS - 1) & 1);                                                                    \
        if (ILV && (NEXT)) {                                                                       \
            _Pragma("unroll") for (int m = 0; m < TM * TN; ++m) {                                  \
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                 \
                if (m < TM + TN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
            }                                                                                      \
        }                                                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                         \
    } while (0)

#pragma unroll
    for (int q = 0; q < NQ; ++q) OPMX_LOADQ(q, 0);
#pragma unroll
    for (int q = 0; q < NQ; ++q) OPMX_DRAINQ(q, 0);
    if (nk > 1) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) OPMX_LOADQ(q, 1);
    }
    __syncthreads();
    OPMX_FRAGS(0, 0, 0);
    {
        static_assert(KS % 2 == 0, "fragment set parity must repeat every k-tile");
        int kt = 0;
        for (; kt + 2 < nk; ++kt) OPMX_ITER(kt, true, true, true);
        if (kt + 1 < nk) {
            OPMX_ITER(kt, true, false, true);
            ++kt;
        }
        OPMX_ITER(kt, false, false, false);
    }
#undef OPMX_ITER
#undef OPMX_MMA
#undef OPMX_FRAGS
#undef OPMX_DRAINQ
#undef OPMX_LOADQ

    // epilogue: acc[i][j][v] is row (v/4)*8 + (lane/32)*4 + v%4, column lane%32 of its 32x32 sub-tile
    const T *be = Bias ? Bias + static_cast<int64_t>(mt.e) * N : nullptr;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < (SWIGLU ? TN / 2 : TN); ++j) {
            const int64_t n = SWIGLU ? n0 + wn * (WTN / 2) + j * 32 + lrow : n0 + wn * WTN + j * 32 + lrow;
            if (n >= ncols) continue;
            const float bg = be ? to_f32(be[n]) : 0.0f;
            const float bu = (SWIGLU && be) ? to_f32(be[ncols + n]) : 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * WTM + i * 32 + (v / 4) * 8 + lk * 4 + (v % 4);
                if (row >= mt.rows) continue;
                float val = acc[i][j][v] + bg;
                if (SWIGLU) {
                    const float up = acc[i][j + TN / 2][v] + bu;
                    val = up * val * sigmoidf_(val);
                }
                Y[(mt.row0 + row) * ncols + n] = from_f32<T>(val);
            }
        }
}

template <typename T, int BM, int BN, int WM, int WN, bool ILV = false>
int tiled_launch(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                 int64_t N, int epilogue, void *Y, hipStream_t s)
{
    constexpr int smem = 2 * (BM + BN) * ROWB;
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    const int64_t ncols = sw ? N / 2 : N;
    const int ntiles_n = static_cast<int>(ceil_div(ncols, sw ? BN / 2 : BN));
    const int ntiles_m = static_cast<int>(max_mtiles(R, E, BM));
    // XCD-grouped order only when the n-tiles split evenly over the 8 XCDs (else some XCDs idle)
    int gnx = ntiles_n % 16 == 0 ? 2 : (ntiles_n % 8 == 0 ? 1 : 0);
    if (const char *v = std::getenv("OPMX_MOE_GEMM_GNX")) gnx = std::atoi(v);   // tuning knob (0: row-major)
    if (gnx != 0 && gnx != 1 && gnx != 2 && gnx != 4 && gnx != 8 && gnx != 16 && gnx != 32) gnx = 0;
    const int64_t nblocks = gnx > 0 ? ceil_div(ntiles_n, 8 * gnx) * ceil_div(ntiles_m, 32 / gnx) * 256
                                    : static_cast<int64_t>(ntiles_n) * ntiles_m;
    dim3 grid(static_cast<unsigned>(nblocks));
    dim3 block(WM * WN * 64);
    static bool attr_done[2] = {false, false};
    if (sw) {
        auto kern = gemm_tiled_kernel<T, BM, BN, WM, WN, true, ILV>;
        if (!attr_done[1]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    smem) != hipSuccess)
                return OPMX_ERR_LAUNCH;
            attr_done[1] = true;
        }
        kern<<<grid, block, smem, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                       static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), ntiles_m, ntiles_n, gnx);
    } else {
        auto kern = gemm_tiled_kernel<T, BM, BN, WM, WN, false, ILV>;
        if (!attr_done[0]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    smem) != hipSuccess)
                return OPMX_ERR_LAUNCH;
            attr_done[0] = true;
        }
        kern<<<grid, block, smem, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                       static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), ntiles_m, ntiles_n, gnx);
    }
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T>
int tiled_impl(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
               int64_t N, int epilogue, int variant, void *Y, hipStream_t s)
{
    // The fixed MFMA / LDS / global-load interleave pays on the 256x256 tiles only.
    switch (variant) {
        case 1: return tiled_launch<T, 256, 256, 2, 2, true>(X, off, W, B, E, R, K, N, epilogue, Y, s);
        case 2: return tiled_launch<T, 256, 128, 2, 2>(X, off, W, B, E, R, K, N, epilogue, Y, s);
        case 3: return tiled_launch<T, 256, 256, 2, 4, true>(X, off, W, B, E, R, K, N, epilogue, Y, s);
        case 4: return tiled_launch<T, 256, 128, 4, 2>(X, off, W, B, E, R, K, N, epilogue, Y, s);
        case 5: return tiled_launch<T, 128, 256, 2, 4>(X, off, W, B, E, R, K, N, epilogue, Y, s);
        default: return tiled_launch<T, 128, 128, 2, 2>(X, off, W, B, E, R, K, N, epilogue, Y, s);
    }
}

}  // namespace

// Requires: dtype f16/bf16, K % 64 == 0, 16-byte aligned X and W, N*K < 2^31.
int launch_gemm_tiled(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                      int64_t K, int64_t N, int dtype, int epilogue, int variant, void *Y, hipStream_t s)
{
    switch (dtype) {
        case OPMX_DTYPE_F16: return tiled_impl<f16>(X, off, W, B, E, R, K, N, epilogue, variant, Y, s);
        case OPMX_DTYPE_BF16: return tiled_impl<bf16>(X, off, W, B, E, R, K, N, epilogue, variant, Y, s);
    }
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
