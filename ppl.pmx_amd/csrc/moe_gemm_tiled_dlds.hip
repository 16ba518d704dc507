// Grouped expert GEMM for gfx950, MFMA-bound regime, direct-to-LDS variant.
//
// Same tiling as moe_gemm_tiled.hip (256x256 output tile of one expert, 8 waves as
// 2x4, 128x64 per wave, v_mfma_f32_32x32x16, fp32 accumulators, optional SwiGLU
// epilogue, tile list derived on the device from expert_offset) but the operand
// tiles never pass through registers: global_load_lds_dwordx4 writes 1 KiB per wave
// instruction straight into LDS (lane l lands at base + 16*l), so staging costs no
// VGPRs, no ds_write and no mid-loop waits.  LDS holds FOUR stages of BK=32
// (32 KiB each); the loads of stage kt+3 are issued while stage kt is consumed, i.e.
// 1.5 k-tiles of 64 ahead of the MFMAs.
//
// LDS layout of a stage: [256 X rows | 256 W rows] x 64 bytes.  16-byte chunk c of
// row r sits at r*64 + ((c ^ ((r>>2)&3)) << 4): sixteen consecutive rows of one
// chunk column cover all sixteen 16-byte bank groups (conflict-free ds_read_b128);
// the XOR is applied by choosing which global chunk a lane fetches.
//
// Synchronisation per k-tile (one barrier): MFMA group 0 -> wait until the loads of
// stage kt+1 have landed (s_waitcnt vmcnt(n), n = younger loads allowed in flight) and
// this wave's fragment reads of stage kt are done -> barrier -> MFMA group 1 while
// the first fragments of stage kt+1 are fetched.  The stage overwritten by the loads
// issued in iteration kt is the one read in iteration kt-1, which every wave left
// before the previous barrier.
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67,
// torch_function/MoeRowParallelLinear.py:47-53, torch_function/SwiGLU.py:15-16.
#include <cstdlib>

#include "moe_gemm.h"

namespace opmx {
namespace {

constexpr int DBK = 32;                // k elements per stage
constexpr int DROWB = DBK * 2;         // 64 bytes per LDS row
constexpr int DSTAGES = 4;

#define OPMX_GPTR(p) ((const void __attribute__((address_space(1))) *)(p))
#define OPMX_LPTR(p) ((void __attribute__((address_space(3))) *)(p))

// Block barrier WITHOUT a memory fence: a fence would have to wait for every in-flight
// direct-to-LDS load (vmcnt(0)) and collapse the multi-stage pipeline.  Ordering is
// explicit instead: the issuing wave waits (vmcnt) for the stage it publishes and for its
// own LDS reads (lgkmcnt) before arriving.
__device__ __forceinline__ void barrier_no_fence()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int N> __device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt immediate");
    if (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (N == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
}

template <typename T, int BM, int BN, int WM, int WN, bool SWIGLU>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tiled_dlds_kernel(const T *__restrict__ X,
                                                                       const int64_t *__restrict__ off,
                                                                       const T *__restrict__ W,
                                                                       const T *__restrict__ Bias, int E,
                                                                       int64_t R, int64_t K, int64_t N,
                                                                       T *__restrict__ Y, int ntiles_m,
                                                                       int ntiles_n)
{
    constexpr int NW = WM * WN;
    constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    constexpr int BNO = SWIGLU ? BN / 2 : BN;
    constexpr int LA = BM / 16 / NW, LB = BN / 16 / NW;   // 1 KiB wave loads per wave per stage
    constexpr int STAGE = (BM + BN) * DROWB;
    static_assert(BM % (16 * NW) == 0 && BN % (16 * NW) == 0, "tile/waves mismatch");
    static_assert(LA + LB == 4, "the vmcnt immediates below assume 4 loads per wave per stage");
    static_assert(!SWIGLU || TN % 2 == 0, "SwiGLU needs an even number of n sub-tiles per wave");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ int64_t s_off[OPMX_MOE_MAX_EXPERTS + 1];

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);
    const int tile_m = blockIdx.x / ntiles_n, tile_n = blockIdx.x % ntiles_n;
    if (tile_m >= ntiles_m) return;
    const MTile mt = find_mtile(off, E, R, BM, tile_m, s_off);
    if (mt.rows == 0) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int64_t n0 = static_cast<int64_t>(tile_n) * BNO;
    const char *xb = reinterpret_cast<const char *>(X + mt.row0 * K);
    const char *wb = reinterpret_cast<const char *>(W + static_cast<int64_t>(mt.e) * N * K);

    // ---- this lane's share of the wave loads: row = 16*(wave*L+i) + lane/4, LDS slot lane%4
    const int lrow4 = lane >> 2, slot = lane & 3;
    uint32_t a_src[LA], b_src[LB];     // byte offsets from xb / wb at k = 0
    int a_lds[LA], b_lds[LB];          // wave-uniform LDS byte offset inside a stage
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = (wave * LA + i) * 16 + lrow4;
        const int r = row < mt.rows ? row : mt.rows - 1;
        const int c = slot ^ ((row >> 2) & 3);
        a_src[i] = static_cast<uint32_t>((r * K + c * 8) * 2);
        a_lds[i] = (wave * LA + i) * 1024;
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = (wave * LB + i) * 16 + lrow4;
        int64_t wrow;
        if (SWIGLU) {
            const int w = row / WTN, jj = row % WTN, half = jj / (WTN / 2);
            int64_t ii = n0 + w * (WTN / 2) + jj % (WTN / 2);
            ii = ii < ncols ? ii : ncols - 1;
            wrow = half * ncols + ii;
        } else {
            wrow = n0 + row < N ? n0 + row : N - 1;
        }
        const int c = slot ^ ((row >> 2) & 3);
        b_src[i] = static_cast<uint32_t>((wrow * K + c * 8) * 2);
        b_lds[i] = BM * DROWB + (wave * LB + i) * 1024;
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int nk = static_cast<int>(K / DBK);
    const int lrow = lane & 31, lk = lane >> 5;
    int fa_off[TM], fb_off[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa_off[i] = (wm * WTM + i * 32 + lrow) * DROWB;
#pragma unroll
    for (int j = 0; j < TN; ++j) fb_off[j] = BM * DROWB + (wn * WTN + j * 32 + lrow) * DROWB;
    const int swz = (lrow >> 2) & 3;   // fragment rows of a lane differ by multiples of 32
    frag fa[2][TM], fb[2][TN];

#define OPMX_ISSUE(KT)                                                                             \
    do {                                                                                           \
        char *st_ = smem + ((KT) % DSTAGES) * STAGE;                                               \
        const int64_t kb_ = static_cast<int64_t>(KT) * (DBK * 2);                                  \
        _Pragma("unroll") for (int i = 0; i < LA; ++i)                                             \
            __builtin_amdgcn_global_load_lds(OPMX_GPTR(xb + kb_ + a_src[i]), OPMX_LPTR(st_ + a_lds[i]), 16, 0, 0); \
        _Pragma("unroll") for (int i = 0; i < LB; ++i)                                             \
            __builtin_amdgcn_global_load_lds(OPMX_GPTR(wb + kb_ + b_src[i]), OPMX_LPTR(st_ + b_lds[i]), 16, 0, 0); \
    } while (0)
#define OPMX_FRAGS(SET, KT, G)                                                                     \
    do {                                                                                           \
        const char *src_ = smem + ((KT) % DSTAGES) * STAGE;                                        \
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
// one k-tile.  ISSUE: there is a tile kt+3 to fetch.  INFLIGHT: loads younger than tile kt+1
// that may still be in flight at the barrier (8, 4 or 0).  NEXT: there is a tile kt+1.
#define OPMX_ITER(KT, ISSUE, INFLIGHT, NEXT)                                                       \
    do {                                                                                           \
        if (ISSUE) OPMX_ISSUE((KT) + 3);                                                           \
        OPMX_FRAGS(1, KT, 1);                                                                      \
        OPMX_MMA(0);                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                         \
        wait_vmcnt<INFLIGHT>();                                                                    \
        barrier_no_fence();                                                                        \
        if (NEXT) OPMX_FRAGS(0, (KT) + 1, 0);                                                      \
        OPMX_MMA(1);                                                                               \
        __builtin_amdgcn_sched_barrier(0);                                                         \
    } while (0)

    // prologue: tiles 0..2 in flight, wait for tile 0
    OPMX_ISSUE(0);
    if (nk > 1) OPMX_ISSUE(1);
    if (nk > 2) OPMX_ISSUE(2);
    if (nk > 2) wait_vmcnt<8>();
    else if (nk > 1) wait_vmcnt<4>();
    else wait_vmcnt<0>();
    barrier_no_fence();
    OPMX_FRAGS(0, 0, 0);
    {
        int kt = 0;
        for (; kt + 3 < nk; ++kt) OPMX_ITER(kt, true, 8, true);
        if (kt + 2 < nk) {
            OPMX_ITER(kt, false, 4, true);
            ++kt;
        }
        if (kt + 1 < nk) {
            OPMX_ITER(kt, false, 0, true);
            ++kt;
        }
        OPMX_ITER(kt, false, 0, false);
    }
#undef OPMX_ITER
#undef OPMX_MMA
#undef OPMX_FRAGS
#undef OPMX_ISSUE

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

template <typename T, bool SW>
int dlds_launch(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                int64_t N, void *Y, hipStream_t s)
{
    constexpr int BM = 256, BN = 256;
    constexpr int smem = DSTAGES * (BM + BN) * DROWB;
    const int64_t ncols = SW ? N / 2 : N;
    const int ntiles_n = static_cast<int>(ceil_div(ncols, SW ? BN / 2 : BN));
    const int ntiles_m = static_cast<int>(max_mtiles(R, E, BM));
    auto kern = gemm_tiled_dlds_kernel<T, BM, BN, 2, 4, SW>;
    static bool attr_done = false;
    if (!attr_done) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                smem) != hipSuccess)
            return OPMX_ERR_LAUNCH;
        attr_done = true;
    }
    kern<<<static_cast<unsigned>(static_cast<int64_t>(ntiles_n) * ntiles_m), 512, smem, s>>>(
        static_cast<const T *>(X), off, static_cast<const T *>(W), static_cast<const T *>(B), E, R, K, N,
        static_cast<T *>(Y), ntiles_m, ntiles_n);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

// Requires: dtype f16/bf16, K % 32 == 0, 16-byte aligned X and W, N*K < 2^31, rows-per-tile * K * 2 < 2^32.
int launch_gemm_tiled_dlds(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                           int64_t K, int64_t N, int dtype, int epilogue, void *Y, hipStream_t s)
{
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    if (dtype == OPMX_DTYPE_F16)
        return sw ? dlds_launch<f16, true>(X, off, W, B, E, R, K, N, Y, s)
                  : dlds_launch<f16, false>(X, off, W, B, E, R, K, N, Y, s);
    if (dtype == OPMX_DTYPE_BF16)
        return sw ? dlds_launch<bf16, true>(X, off, W, B, E, R, K, N, Y, s)
                  : dlds_launch<bf16, false>(X, off, W, B, E, R, K, N, Y, s);
    return OPMX_ERR_UNSUPPORTED;
}

}  // namespace opmx
