// Grouped expert GEMM for fp32 tensors on the fp32 matrix units of gfx950.
//
//   Y[r, :] = X[r, :] W[e]^T (+ B[e])   for off[e] <= r < off[e+1]
//
// float32 is the first type the reference's operators list (docs/operators/MoeColumnParallelLinear.md:73)
// and the type of its CPU-runnable configuration.  A workgroup of four waves owns BM rows of one
// expert times 128 rows of W[e] (tiles never straddle experts; the row tile comes from
// expert_offset on the device), walks K in tiles of 32 floats through two LDS stages -- 16-byte
// global loads, coalesced along K, one register stage ahead of the LDS stores, one barrier per
// k-tile -- and accumulates with v_mfma_f32_16x16x4_f32: W is the A operand, X the B operand, so
// a lane ends up with four consecutive output columns of one row.  A lane reads four consecutive
// k values of its row with one 16-byte LDS read and feeds them to four MFMAs; the k values of
// the four lane groups interleave, the same way for both operands, which only reorders the sum.
// fp32 accumulation in the matrix unit, no rounding before the store.  Optional SwiGLU epilogue:
// a wave's 32 W rows are then 16 gate rows and the 16 up rows of the same output columns.
// Needs K % 4 == 0 and 16-byte aligned X and W; other fp32 shapes take the shape-agnostic kernel.
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67,
// torch_function/MoeRowParallelLinear.py:47-53, torch_function/SwiGLU.py:15-16.
#include "moe_gemm.h"

namespace opmx {
namespace {

constexpr int FBN = 128;               // W rows per tile (4 waves x 32)
constexpr int FBK = 32;                // floats per k-tile (128 bytes per row)
constexpr int FLD = FBK + 4;           // LDS row pitch in floats: 16-byte reads of 8 consecutive rows hit 8 bank groups
constexpr int FCH = FBK / 4;           // 16-byte chunks per row and k-tile

template <int BM, bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float *__restrict__ X, const int64_t *__restrict__ off,
                                                       const float *__restrict__ W, const float *__restrict__ Bias,
                                                       int E, int64_t R, int64_t K, int64_t N, float *__restrict__ Y,
                                                       const int32_t *__restrict__ rt, int64_t xrows)
{
    constexpr int TMS = BM / 16;                       // 16-row sub-tiles of X per wave (a wave takes all BM rows)
    constexpr int BNO = SWIGLU ? FBN / 2 : FBN;        // output columns per tile
    constexpr int LA = BM * FCH / 256, LB = FBN * FCH / 256;   // 16-byte loads per thread and k-tile
    static_assert(BM % 32 == 0, "whole loads per thread");
    extern __shared__ __attribute__((aligned(16))) float lds[];   // two stages of (BM + FBN) rows

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);
    const MTile mt = find_mtile(off, E, R, BM, blockIdx.y);
    if (mt.rows == 0) return;
    const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BNO;
    const float *We = W + static_cast<int64_t>(mt.e) * N * K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // this thread's loads: chunk tid % 8 of tile rows tid / 8 + 32 * i
    const int lc = tid % FCH, lr = tid / FCH;
    const float *xsrc[LA];
    bool xok[LA];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = lr + 32 * i;
        xok[i] = row < mt.rows;
        const int64_t r = mt.row0 + (xok[i] ? row : 0);
        xsrc[i] = X + (rt ? gathered_row(rt, xrows, r) : r) * K + lc * 4;
    }
    const float *wsrc[LB];
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = lr + 32 * i;            // tile row: wave row / 32, inside it 16 gate + 16 up rows with SWIGLU
        int64_t wrow;
        if (SWIGLU) {
            const int w = row / 32, jj = row % 32;
            int64_t c = n0 + w * 16 + jj % 16;
            c = c < ncols ? c : ncols - 1;
            wrow = (jj / 16) * ncols + c;
        } else {
            wrow = n0 + row < N ? n0 + row : N - 1;    // rows past the matrix repeat the last one (never stored)
        }
        wsrc[i] = We + wrow * K + lc * 4;
    }
    constexpr int STAGE = (BM + FBN) * FLD;
    const int xdst = lr * FLD + lc * 4, wdst = (BM + lr) * FLD + lc * 4;

    float4_t acc[2][TMS];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int nk = static_cast<int>((K + FBK - 1) / FBK);
    float4_t rx[LA], rw[LB];
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int kt) {
        const int64_t k0 = static_cast<int64_t>(kt) * FBK;
        const bool kin = k0 + lc * 4 < K;           // K % 4 == 0: a chunk lies inside K or outside as a whole
#pragma unroll
        for (int i = 0; i < LA; ++i)
            rx[i] = (kin && xok[i]) ? *reinterpret_cast<const float4_t *>(xsrc[i] + k0) : zero4;
#pragma unroll
        for (int i = 0; i < LB; ++i) rw[i] = kin ? *reinterpret_cast<const float4_t *>(wsrc[i] + k0) : zero4;
    };
    auto park = [&](int buf) {
        float *st = lds + buf * STAGE;
#pragma unroll
        for (int i = 0; i < LA; ++i) *reinterpret_cast<float4_t *>(st + xdst + 32 * i * FLD) = rx[i];
#pragma unroll
        for (int i = 0; i < LB; ++i) *reinterpret_cast<float4_t *>(st + wdst + 32 * i * FLD) = rw[i];
    };

    const int fr = lane & 15, fg = lane >> 4;
    fetch(0);
    park(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        if (kt + 1 < nk) fetch(kt + 1);
        const float *st = lds + (kt & 1) * STAGE;
        const float *xs = st + fr * FLD + fg * 4;
        const float *ws = st + (BM + wave * 32 + fr) * FLD + fg * 4;
#pragma unroll
        for (int h = 0; h < FBK / 16; ++h) {
            float4_t a[2], b[TMS];
#pragma unroll
            for (int j = 0; j < 2; ++j) a[j] = *reinterpret_cast<const float4_t *>(ws + j * 16 * FLD + h * 16);
#pragma unroll
            for (int i = 0; i < TMS; ++i) b[i] = *reinterpret_cast<const float4_t *>(xs + i * 16 * FLD + h * 16);
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < TMS; ++i)
                        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j][v], b[i][v], acc[j][i], 0, 0, 0);
        }
        if (kt + 1 < nk) park((kt + 1) & 1);
        __syncthreads();
    }

    // acc[j][i][v]: X row i*16 + fr, W row wave*32 + j*16 + fg*4 + v of the tile
    const float *be = Bias ? Bias + static_cast<int64_t>(mt.e) * N : nullptr;
    const bool vec = ncols % 4 == 0 && reinterpret_cast<uintptr_t>(Y) % 16 == 0;
#pragma unroll
    for (int i = 0; i < TMS; ++i) {
        const int row = i * 16 + fr;
        if (row >= mt.rows) continue;
        float *yrow = Y + (mt.row0 + row) * ncols;
#pragma unroll
        for (int j = 0; j < (SWIGLU ? 1 : 2); ++j) {
            const int64_t n = n0 + (SWIGLU ? wave * 16 : wave * 32 + j * 16) + fg * 4;
            if (n >= ncols) continue;
            float val[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t nn = n + v < ncols ? n + v : ncols - 1;
                float g = acc[j][i][v] + (be ? be[nn] : 0.0f);
                if (SWIGLU) {
                    const float up = acc[1][i][v] + (be ? be[ncols + nn] : 0.0f);
                    g = up * g * sigmoidf_(g);
                }
                val[v] = g;
            }
            if (vec && n + 3 < ncols) {
                *reinterpret_cast<float4_t *>(yrow + n) = float4_t{val[0], val[1], val[2], val[3]};
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < ncols) yrow[n + v] = val[v];
            }
        }
    }
}


// Few rows per expert (decode-sized calls): the job is to stream every active expert's weights once,
// and with 128 W rows per workgroup a short N leaves most of the chip idle behind a long serial walk
// over K (8 experts x 1024 output columns x 16 rows each: 96 workgroups with 88 k-tiles each).  Here a
// workgroup owns 32 rows of one expert times 32 rows of W[e] and its four waves split K: wave w walks
// the k-tiles w, w + 4, ... on its own, staging them through wave-private LDS (coalesced 16-byte
// loads, two stages, no block barrier in the loop), and the four partial sums meet in LDS after the
// loop, added in wave order (so the result does not depend on timing).  Four times the workgroups,
// a quarter of the serial chain.  With SWIGLU the 32 W rows are 16 gate rows and their 16 up rows.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_f32_splitk_kernel(const float *__restrict__ X, const int64_t *__restrict__ off,
                                                              const float *__restrict__ W, const float *__restrict__ Bias,
                                                              int E, int64_t R, int64_t K, int64_t N, float *__restrict__ Y,
                                                              const int32_t *__restrict__ rt, int64_t xrows)
{
    constexpr int BM = 32, WR = 32, TMS = BM / 16;
    constexpr int BNO = SWIGLU ? WR / 2 : WR;          // output columns per workgroup
    constexpr int STAGE = (BM + WR) * FLD;             // floats per wave and stage
    constexpr int NLD = (BM + WR) * FCH / 64;          // 16-byte loads per lane and k-tile (8)
    __shared__ __attribute__((aligned(16))) float lds[4 * 2 * STAGE];   // 4 waves x 2 stages; reused for the partial sums

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);
    const MTile mt = find_mtile(off, E, R, BM, blockIdx.y);
    if (mt.rows == 0) return;
    const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BNO;
    const float *We = W + static_cast<int64_t>(mt.e) * N * K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float *mine = lds + wave * 2 * STAGE;

    // this lane's loads: chunk lane % 8 of rows lane / 8 + 8 * i; rows [0, 32) are X rows, [32, 64) W rows
    const int lc = lane % FCH, lr = lane / FCH;
    const float *src[NLD];
    bool ok[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int row = lr + 8 * i;
        if (row < BM) {
            ok[i] = row < mt.rows;
            const int64_t r = mt.row0 + (ok[i] ? row : 0);
            src[i] = X + (rt ? gathered_row(rt, xrows, r) : r) * K + lc * 4;
        } else {
            const int wr = row - BM;
            int64_t wrow;
            if (SWIGLU) {
                int64_t c = n0 + wr % 16;
                c = c < ncols ? c : ncols - 1;
                wrow = (wr / 16) * ncols + c;
            } else {
                wrow = n0 + wr < N ? n0 + wr : N - 1;
            }
            ok[i] = true;
            src[i] = We + wrow * K + lc * 4;
        }
    }
    const int dst = lr * FLD + lc * 4;

    float4_t acc[2][TMS];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i) acc[j][i] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int nk = static_cast<int>((K + FBK - 1) / FBK);
    float4_t reg[NLD];
    const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    auto fetch = [&](int kt) {
        const int64_t k0 = static_cast<int64_t>(kt) * FBK;
        const bool kin = k0 + lc * 4 < K;
#pragma unroll
        for (int i = 0; i < NLD; ++i) reg[i] = (kin && ok[i]) ? *reinterpret_cast<const float4_t *>(src[i] + k0) : zero4;
    };
    auto park = [&](int buf) {
        float *st = mine + buf * STAGE;
#pragma unroll
        for (int i = 0; i < NLD; ++i) *reinterpret_cast<float4_t *>(st + dst + 8 * i * FLD) = reg[i];
    };
    const int fr = lane & 15, fg = lane >> 4;
    int buf = 0;
    if (wave < nk) {
        fetch(wave);
        park(0);
    }
    for (int kt = wave; kt < nk; kt += 4, buf ^= 1) {
        if (kt + 4 < nk) fetch(kt + 4);
        __builtin_amdgcn_wave_barrier();             // the wave's own LDS writes above, its reads below: program order
        const float *st = mine + buf * STAGE;
        const float *xs = st + fr * FLD + fg * 4;
        const float *ws = st + (BM + fr) * FLD + fg * 4;
#pragma unroll
        for (int h = 0; h < FBK / 16; ++h) {
            float4_t a[2], b[TMS];
#pragma unroll
            for (int j = 0; j < 2; ++j) a[j] = *reinterpret_cast<const float4_t *>(ws + j * 16 * FLD + h * 16);
#pragma unroll
            for (int i = 0; i < TMS; ++i) b[i] = *reinterpret_cast<const float4_t *>(xs + i * 16 * FLD + h * 16);
#pragma unroll
            for (int v = 0; v < 4; ++v)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < TMS; ++i)
                        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j][v], b[i][v], acc[j][i], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
        if (kt + 4 < nk) park(buf ^ 1);
    }

    // the four partial sums: part[wave][j][i][lane], added in wave order by the wave that stores the sub-tile
    __syncthreads();
    float *part = lds;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i)
            *reinterpret_cast<float4_t *>(part + (((wave * 2 + j) * TMS + i) * 64 + lane) * 4) = acc[j][i];
    __syncthreads();
    // wave w stores the sub-tile (j, i) = (w / TMS, w % TMS); with SWIGLU waves 0 .. TMS-1 store row block i = w
    const int oi = wave % TMS, oj = SWIGLU ? 0 : wave / TMS;
    if (SWIGLU && wave >= TMS) return;
    float4_t sum[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        sum[j] = zero4;
        if (j == oj || SWIGLU)
#pragma unroll
            for (int w = 0; w < 4; ++w)
                sum[j] += *reinterpret_cast<const float4_t *>(part + (((w * 2 + j) * TMS + oi) * 64 + lane) * 4);
    }
    const int row = oi * 16 + fr;
    if (row >= mt.rows) return;
    const int64_t n = n0 + (SWIGLU ? 0 : oj * 16) + fg * 4;
    if (n >= ncols) return;
    const float *be = Bias ? Bias + static_cast<int64_t>(mt.e) * N : nullptr;
    float *yrow = Y + (mt.row0 + row) * ncols;
    float val[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int64_t nn = n + v < ncols ? n + v : ncols - 1;
        float g = sum[oj][v] + (be ? be[nn] : 0.0f);
        if (SWIGLU) {
            const float up = sum[1][v] + (be ? be[ncols + nn] : 0.0f);
            g = up * g * sigmoidf_(g);
        }
        val[v] = g;
    }
    if (ncols % 4 == 0 && reinterpret_cast<uintptr_t>(Y) % 16 == 0 && n + 3 < ncols) {
        *reinterpret_cast<float4_t *>(yrow + n) = float4_t{val[0], val[1], val[2], val[3]};
    } else {
#pragma unroll
        for (int v = 0; v < 4; ++v)
            if (n + v < ncols) yrow[n + v] = val[v];
    }
}

int f32_splitk_launch(const float *X, const int64_t *off, const float *W, const float *B, int E, int64_t R, int64_t K,
                      int64_t N, int epilogue, float *Y, hipStream_t s, RowGather g)
{
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    const int64_t ncols = sw ? N / 2 : N;
    const dim3 grid(static_cast<unsigned>(ceil_div(ncols, sw ? 16 : 32)), static_cast<unsigned>(max_mtiles(R, E, 32)));
    if (sw) gemm_f32_splitk_kernel<true><<<grid, 256, 0, s>>>(X, off, W, B, E, R, K, N, Y, g.index, g.x_rows);
    else gemm_f32_splitk_kernel<false><<<grid, 256, 0, s>>>(X, off, W, B, E, R, K, N, Y, g.index, g.x_rows);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <int BM>
int f32_launch(const float *X, const int64_t *off, const float *W, const float *B, int E, int64_t R, int64_t K, int64_t N,
               int epilogue, float *Y, hipStream_t s, RowGather g)
{
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    const int64_t ncols = sw ? N / 2 : N;
    constexpr int smem = 2 * (BM + FBN) * FLD * static_cast<int>(sizeof(float));
    const dim3 grid(static_cast<unsigned>(ceil_div(ncols, sw ? FBN / 2 : FBN)), static_cast<unsigned>(max_mtiles(R, E, BM)));
    static std::atomic<uint64_t> attr_done[2];
    if (sw) {
        auto kern = gemm_f32_kernel<BM, true>;
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done[1])) return OPMX_ERR_LAUNCH;
        kern<<<grid, 256, smem, s>>>(X, off, W, B, E, R, K, N, Y, g.index, g.x_rows);
    } else {
        auto kern = gemm_f32_kernel<BM, false>;
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done[0])) return OPMX_ERR_LAUNCH;
        kern<<<grid, 256, smem, s>>>(X, off, W, B, E, R, K, N, Y, g.index, g.x_rows);
    }
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace

// Requires K % 4 == 0 and 16-byte aligned X and W.
int launch_gemm_f32(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                    int64_t N, int epilogue, int64_t rows_hint, void *Y, hipStream_t s, RowGather g)
{
    const float *x = static_cast<const float *>(X), *w = static_cast<const float *>(W), *b = static_cast<const float *>(B);
    float *y = static_cast<float *>(Y);
    // Up to 128 rows per expert (twice the mean), or whenever 128 x 128 tiles would not fill the chip
    // twice: 32-row tiles whose waves split K -- the weights stream through once per row tile (from the
    // L2 or the memory-side cache after the first) and the chip is full whatever N is.  Measured against
    // the 128-column forms (8 experts, even rows; gate/up | down): hidden 1024 / ffn 2816: 16 rows per
    // expert 49 -> 48 | 78 -> 26 us, 32 rows 139 -> 54 | 213 -> 27, 64 rows 146 -> 94 | 212 -> 39, 128 rows
    // 148 -> 173 (kept on 128-row tiles) | 212 -> 75, 256 rows 282 -> 320 (kept) | 213 -> 144; hidden 4096 /
    // ffn 14336: one token 139 -> 119 | 377 -> 110, 4 rows 874 -> 838 | 458 -> 368, 32 rows 1898 -> 849 |
    // 1072 -> 405, 64 rows 1928 -> 1665 | 1064 -> 712, 128 rows 2057 -> 3327 | 1061 -> 1353 (both kept).
    // OPMX_MOE_GEMM_F32_VARIANT: 0 never, 1 always.
    const int v = option(kOptF32Variant);
    const int64_t ncols = epilogue == OPMX_EPILOGUE_SWIGLU ? N / 2 : N;
    const int64_t wgs128 = ceil_div(ncols, epilogue == OPMX_EPILOGUE_SWIGLU ? FBN / 2 : FBN) * max_mtiles(R, E, 128);
    if (v == 1 || (v != 0 && K >= 4 * FBK && (rows_hint <= 128 || wgs128 < 512)))
        return f32_splitk_launch(x, off, w, b, E, R, K, N, epilogue, y, s, g);
    if (rows_hint <= 32) return f32_launch<32>(x, off, w, b, E, R, K, N, epilogue, y, s, g);
    return f32_launch<128>(x, off, w, b, E, R, K, N, epilogue, y, s, g);
}

}  // namespace opmx
