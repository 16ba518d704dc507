// Grouped expert GEMM for gfx950, MFMA-bound regime (many rows per expert).
//
//   Y[r, :] = X[r, :] W[e]^T (+ B[e])   for off[e] <= r < off[e+1]
//
// X [R,K] and W[e] [N,K] are both K-contiguous, so MFMA fragments are 16-byte LDS reads.
// A workgroup owns a BM x BN output tile of ONE expert (tiles never straddle experts; the
// tile list is derived on the device from expert_offset, no host sync), streams BK=64
// k-tiles of X and W through XOR-swizzled LDS and accumulates in fp32 with
// v_mfma_f32_16x16x32 (measured ~10% more flops at the same board power than 32x32x16 on
// random operands: a quarter of the accumulator registers move per instruction).  W is the
// A operand and X the B operand, so a lane holds four consecutive output COLUMNS of a row.
// Optional SwiGLU epilogue on the accumulators (gate rows i and up rows N/2+i of W are
// placed in the same lane by the W-tile row order).
//
// Two kernels share the tile order, LDS layout and epilogues:
//   gemm_tiled_dlds_kernel  256x256 tile, 4 waves, operands loaded straight into LDS, the
//                           fragments of a whole k-tile held in registers.  Default from 128
//                           mean rows per expert on.
//   gemm_tiled_kernel       operands staged through registers (global -> VGPR -> LDS), any
//                           BM x BN / wave layout; 128x128 tiles are the default below that.
// Semantics: torch_function/MoeColumnParallelLinear.py:61-67,
// torch_function/MoeRowParallelLinear.py:47-53, torch_function/SwiGLU.py:15-16.
#include <cstdlib>

#include "moe_gemm.h"

namespace opmx {
namespace {

constexpr int BK = 64;                 // k elements per LDS tile (128 bytes per row)
constexpr int ROWB = BK * 2;           // bytes per LDS row
constexpr int CH = ROWB / 16;          // 16-byte chunks per row (8)

// Byte offset of 16-byte chunk `chunk` of tile row `row`: 16 consecutive rows of one chunk
// column land in sixteen different 16-byte bank groups (conflict-free b128 fragment reads).
__device__ __forceinline__ int lds_off(int row, int chunk) { return row * ROWB + ((chunk ^ ((row >> 1) & 7)) << 4); }

// What a workgroup knows about the experts, in LDS: the offsets clamped into [0, R] (a corrupt
// offset can never send a store outside Y; a segment that ends before it starts counts as empty)
// and the running number of row tiles in front of every expert.  Looking a tile up is then a
// search in `pref`, done by the lanes of a wave together (find_expert) instead of a walk over the
// experts by every thread: with 64 experts that walk cost a microsecond per tile, with 256 four.
struct ExpertTable {
    int64_t off[OPMX_MOE_MAX_EXPERTS + 1];
    int pref[OPMX_MOE_MAX_EXPERTS + 4];     // pref[e] = row tiles of experts < e; pref[E ... 256] = all of them
};

// Fills the table for row tiles of height BM.  Nothing to do for a dense GEMM (off == nullptr).
// Every thread must call it: it contains block barriers.
__device__ __forceinline__ void stage_offsets(const int64_t *__restrict__ off, int E, int64_t R, int BM, ExpertTable &tab)
{
    static_assert(OPMX_MOE_MAX_EXPERTS <= 4 * 64, "four experts per lane");
    if (off == nullptr) return;
    for (int i = threadIdx.x; i <= E; i += blockDim.x) {
        const int64_t v = off[i];
        tab.off[i] = v < 0 ? 0 : (v > R ? R : v);
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x, sh = 31 - __builtin_clz(BM);    // BM is a power of two
        int m[4], tot = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = lane * 4 + q;
            const int64_t rows = e < E ? tab.off[e + 1] - tab.off[e] : 0;
            m[q] = rows > 0 ? static_cast<int>((rows + BM - 1) >> sh) : 0;
            tot += m[q];
        }
        int incl = tot;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
        }
        int run = incl - tot;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            tab.pref[lane * 4 + q] = run;
            run += m[q];
        }
        if (lane == 63) tab.pref[256] = incl;
    }
    __syncthreads();
}

// Number of row tiles of height BM over all experts: sum of ceil(rows_e / BM).
__device__ __forceinline__ int count_mtiles(bool grouped, const ExpertTable &tab, int E, int64_t R, int BM)
{
    const int sh = 31 - __builtin_clz(BM);       // BM is a power of two: shifts, not 64-bit divisions
    if (!grouped) return static_cast<int>((R + BM - 1) >> sh);
    return __builtin_amdgcn_readfirstlane(tab.pref[256]);
}

// The expert that owns row tile `tile_m` (counted over all experts in expert order), or -1.
// Whole waves, converged; the answer is wave-uniform.
__device__ __forceinline__ int find_expert(int tile_m, const ExpertTable &tab)
{
    const int lane = threadIdx.x & 63;
    int p[5];
#pragma unroll
    for (int q = 0; q < 5; ++q) p[q] = tab.pref[lane * 4 + q];
    const uint64_t owner = __ballot(tile_m >= p[0] && tile_m < p[4]);
    if (tile_m < 0 || owner == 0) return -1;
    const int src = __ffsll(static_cast<long long>(owner)) - 1;
    const int q = tile_m < p[1] ? 0 : (tile_m < p[2] ? 1 : (tile_m < p[3] ? 2 : 3));
    return __builtin_amdgcn_readlane(lane * 4 + q, src);
}

// Linear tile id -> (row tile, column tile) over the row tiles of all experts strung together;
// mtiles is the actual number of row tiles.  Workgroups are handed to the 8 XCDs round-robin by
// linear id and each XCD has its own L2, so the order of the ids decides which tiles share an L2.
//   gnx = 4: rounds of 16 x 16 tiles, XCDs as 2 (m) x 4 (n), each a compact 8 x 4 sub-block (a
//            third less L2 fill traffic than 16 x 2).  The last mtiles % 16 row tiles would leave
//            XCDs idle in that layout; XCD j takes their column tiles [j*ntiles_n/8, (j+1)*ntiles_n/8),
//            walking m fastest.  ntiles_n % 16 == 0.  Kept as the comparison point of the
//            expert-major order below, which replaced it.
//   gnx = 0: plain row-major order, n fastest.
// Ids that name no tile come back with tile_m >= mtiles.
__device__ __forceinline__ void map_tile(int lin, int gnx, int mtiles, int ntiles_n, int &tile_m, int &tile_n)
{
    const int xcd = lin & 7, sl = (lin >> 3) & 31, round = lin >> 8;
    if (gnx == 4) {
        const int cols16 = ntiles_n / 16, full = mtiles / 16, rem = mtiles % 16;
        const int ids_full = full * cols16 * 256;
        if (lin < ids_full) {
            tile_m = (round / cols16) * 16 + (xcd >> 2) * 8 + (sl & 7);
            tile_n = (round % cols16) * 16 + (xcd & 3) * 4 + (sl >> 3);
        } else {
            const int s = (lin - ids_full) >> 3, cols = ntiles_n / 8;
            if (rem > 0 && s < rem * cols) {
                tile_m = full * 16 + s % rem;
                tile_n = xcd * cols + s / rem;
            } else {
                tile_m = mtiles;
                tile_n = 0;
            }
        }
    } else {
        tile_m = lin / ntiles_n;
        tile_n = lin % ntiles_n;
    }
}

// Row tile tile_m (counted over all experts in expert order) -> expert and row range.
// mt.rows == 0 when there is no such tile.  tab: see stage_offsets (unused when `grouped` is
// false: one expert owns [0, R)).
__device__ __forceinline__ void row_tile(int tile_m, bool grouped, const ExpertTable &tab, int E, int64_t R, int BM,
                                         MTile &mt)
{
    mt.e = 0;
    mt.rows = 0;
    mt.row0 = 0;
    if (tile_m < 0) return;
    if (!grouped) {
        mt.row0 = static_cast<int64_t>(tile_m) * BM;
        const int64_t left = R - mt.row0;
        mt.rows = left <= 0 ? 0 : static_cast<int>(left < BM ? left : BM);
        return;
    }
    const int e = find_expert(tile_m, tab);
    if (e < 0) return;
    const int64_t row0 = tab.off[e] + static_cast<int64_t>(tile_m - tab.pref[e]) * BM, left = tab.off[e + 1] - row0;
    // block-uniform by construction; say so to the compiler (scalar registers)
    mt.e = e;
    mt.row0 = (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0 >> 32))) << 32) |
              static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0)));
    mt.rows = __builtin_amdgcn_readfirstlane(static_cast<int>(left < BM ? left : BM));
}

// Expert-major order (gnx = 8; ntiles_n % 8 == 0).  The orders above lay their XCD sub-blocks
// over the row tiles of all experts strung together, so a sub-block of 8 row tiles usually
// spans several experts and the workgroups in it share W-tiles only with the rows of their own
// expert: with ragged experts (4 full row tiles and a nearly empty fifth, say) the L2 hit rate
// falls from 74 % to 57-65 % and the HBM reads grow by half.  Here the ids go expert by expert,
// and inside an expert with m row tiles:
//  - every 16 row tiles form a band the XCDs share as 2 (rows) x 4 (columns): XCD x owns rows
//    8*(x/4) .. +7 of the band and the column tiles [(x%4)*C4, +C4), C4 = ntiles_n / 4, and walks
//    its columns with the 8 rows fastest.  Per round of 256 tiles the chip then works on 16 row
//    tiles x 16 column tiles, each XCD on 8 x 4 (as in the gnx = 4 order), and the band's X rows
//    stay in the memory-side cache while the columns go by;
//  - the m % 16 rows left over are walked by all XCDs together: XCD x owns the column tiles
//    [x*C, +C), C = ntiles_n / 8, in row groups of 8 (the last one smaller): for each group, for
//    each column, the rows of the group.  Its 32 resident workgroups cover h rows x 32/h columns
//    (h = 8, or what is left): each W-tile is shared by h of them, each X-tile by 32/h.
// Every XCD gets exactly an eighth of every expert, and the ids [0, sum m_e * ntiles_n) are
// exactly the tiles.
__device__ __forceinline__ void locate_expert_major(int64_t lin, bool grouped, const ExpertTable &tab, int E, int64_t R,
                                                    int BM, int ntiles_n, MTile &mt, int &tile_n)
{
    mt.e = 0;
    mt.rows = 0;
    mt.row0 = 0;
    tile_n = 0;
    const int sh = 31 - __builtin_clz(BM);
    const uint32_t C = static_cast<uint32_t>(ntiles_n) >> 3;
    // expert e owns the ids [pref[e] * ntiles_n, pref[e+1] * ntiles_n): its row tiles times all columns
    int e = 0;
    uint32_t m, l;
    int64_t prev = 0, hi = R;
    if (grouped) {
        if (lin >= (int64_t{1} << 31)) return;
        const uint32_t g = static_cast<uint32_t>(lin) / static_cast<uint32_t>(ntiles_n);
        e = find_expert(static_cast<int>(g), tab);
        if (e < 0) return;
        const uint32_t first = static_cast<uint32_t>(tab.pref[e]);
        m = static_cast<uint32_t>(tab.pref[e + 1]) - first;
        l = static_cast<uint32_t>(lin) - first * static_cast<uint32_t>(ntiles_n);
        prev = tab.off[e];
        hi = tab.off[e + 1];
    } else {
        m = static_cast<uint32_t>((R + BM - 1) >> sh);
        if (lin >= static_cast<int64_t>(m) * ntiles_n) return;
        l = static_cast<uint32_t>(lin);
    }
    uint32_t row, col;
    const uint32_t band = 16u * static_cast<uint32_t>(ntiles_n), bands = m >> 4;
    if (l < bands * band) {
        const uint32_t b = l / band, l2 = l - b * band, xcd = l2 & 7, s = l2 >> 3;
        row = b * 16 + (xcd >> 2) * 8 + (s & 7);
        col = (xcd & 3) * (2 * C) + (s >> 3);
    } else {
        l -= bands * band;
        const uint32_t mr = m - 16 * bands, xcd = l & 7, s = l >> 3;   // s in [0, mr*C)
        const uint32_t full = mr >> 3, per_group = 8 * C;
        uint32_t rg = s / per_group, h = 8;
        if (rg >= full) {
            rg = full;
            h = mr - 8 * full;
        }
        const uint32_t t = s - rg * per_group, c = t / h;
        row = 16 * bands + rg * 8 + (t - c * h);
        col = xcd * C + c;
    }
    const int64_t row0 = prev + static_cast<int64_t>(row) * BM, left = hi - row0;
    // block-uniform by construction; say so to the compiler (scalar registers)
    tile_n = __builtin_amdgcn_readfirstlane(static_cast<int>(col));
    mt.e = __builtin_amdgcn_readfirstlane(e);
    mt.row0 = (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0 >> 32))) << 32) |
              static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0)));
    mt.rows = __builtin_amdgcn_readfirstlane(static_cast<int>(left < BM ? left : BM));
}

// Row-partition order (gnx = 16), for column-tile counts that do not divide by 8 (11 column tiles
// of the fine-grained gate/up GEMM): XCD x (ids = x mod 8) owns the row tiles
// [x*mtiles/8, (x+1)*mtiles/8) with ALL their column tiles, and walks them four rows at a time:
// for each group of four rows, for each column, the rows of the group -- its 32 resident
// workgroups cover 4 rows x 8 columns.  Every expert's W is read by the one or two XCDs that own
// its rows (in row-major order all eight read all of it).  XCDs own mtiles/8 row tiles rounded
// down or up, so up to 8 * ntiles_n ids past the shorter ones name no tile (tile_m >= mtiles).
__device__ __forceinline__ void map_row_partition(int64_t lin, int mtiles, int ntiles_n, int &tile_m, int &tile_n)
{
    const uint32_t xcd = static_cast<uint32_t>(lin) & 7, s = static_cast<uint32_t>(lin >> 3);
    const uint32_t lo = xcd * static_cast<uint32_t>(mtiles) / 8, hi = (xcd + 1) * static_cast<uint32_t>(mtiles) / 8;
    const uint32_t rows = hi - lo, per_group = 4u * static_cast<uint32_t>(ntiles_n);
    tile_m = mtiles;
    tile_n = 0;
    if (s >= rows * static_cast<uint32_t>(ntiles_n)) return;
    const uint32_t grp = s / per_group, t = s - grp * per_group;
    const uint32_t h = rows - 4 * grp < 4 ? rows - 4 * grp : 4;
    const uint32_t c = t / h;
    tile_m = static_cast<int>(lo + 4 * grp + (t - c * h));
    tile_n = static_cast<int>(c);
}

// Expert-grouped partition (gnx = 32), for many small experts (a few row tiles each).  All tiles
// are strung together expert by expert and, inside an expert, in row groups of up to 8 row tiles:
// for each group, for each column tile, the rows of the group.  XCD x (ids = x mod 8) owns the
// contiguous eighth [x*ttot/8, (x+1)*ttot/8) of that string, so its 32 resident workgroups cover
// all m row tiles of one expert times 32/m column tiles: every W-tile is shared by all rows of its
// expert and fetched by one XCD, the expert's X rows by that XCD alone, and the XCDs are balanced to
// one tile.  (The expert-major order gives every XCD an eighth of every expert: with two or three
// row tiles per expert an XCD's workgroups then sit in a dozen experts at once and every XCD
// fetches every X row.)  Up to 7 ids past the end name no tile.  Grouped launches only.
__device__ __forceinline__ void locate_expert_grouped(int64_t lin, const ExpertTable &tab, int BM, int mtiles, int ntiles_n,
                                                      MTile &mt, int &tile_n)
{
    mt.e = 0;
    mt.rows = 0;
    mt.row0 = 0;
    tile_n = 0;
    const uint64_t ttot = static_cast<uint64_t>(mtiles) * static_cast<uint32_t>(ntiles_n);
    const uint32_t xcd = static_cast<uint32_t>(lin) & 7;
    const uint64_t j = static_cast<uint64_t>(lin) >> 3, lo = xcd * ttot / 8, hi = (xcd + 1) * ttot / 8;
    if (lin < 0 || j >= hi - lo) return;
    const uint32_t g = static_cast<uint32_t>(lo + j), nt = static_cast<uint32_t>(ntiles_n);
    const int e = find_expert(static_cast<int>(g / nt), tab);
    if (e < 0) return;
    const uint32_t first = static_cast<uint32_t>(tab.pref[e]), m = static_cast<uint32_t>(tab.pref[e + 1]) - first;
    const uint32_t l = g - first * nt, per_group = 8 * nt, full = m >> 3;
    uint32_t rg = l / per_group, h = 8;
    if (rg >= full) {
        rg = full;
        h = m - 8 * full;
    }
    const uint32_t t = l - rg * per_group, c = t / h, row = rg * 8 + (t - c * h);
    const int64_t row0 = tab.off[e] + static_cast<int64_t>(row) * BM, left = tab.off[e + 1] - row0;
    tile_n = __builtin_amdgcn_readfirstlane(static_cast<int>(c));
    mt.e = __builtin_amdgcn_readfirstlane(e);
    mt.row0 = (static_cast<int64_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0 >> 32))) << 32) |
              static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(row0)));
    mt.rows = __builtin_amdgcn_readfirstlane(static_cast<int>(left < BM ? left : BM));
}

// Linear tile id -> tile, in whichever order gnx names.  mt.rows == 0: the id names no work.
__device__ __forceinline__ void locate_any(int64_t lin, int gnx, int mtiles, int ntiles_n, bool grouped,
                                           const ExpertTable &s_off, int E, int64_t R, int BM, MTile &mt, int &tile_n)
{
    if (gnx == 8) {
        locate_expert_major(lin, grouped, s_off, E, R, BM, ntiles_n, mt, tile_n);
    } else if (gnx == 32 && grouped) {
        locate_expert_grouped(lin, s_off, BM, mtiles, ntiles_n, mt, tile_n);
    } else if (gnx == 16 || gnx == 32) {
        int tile_m;
        map_row_partition(lin, mtiles, ntiles_n, tile_m, tile_n);
        if (tile_m >= mtiles || tile_n >= ntiles_n) tile_m = -1;
        row_tile(tile_m, grouped, s_off, E, R, BM, mt);
    } else {
        int tile_m;
        map_tile(static_cast<int>(lin), gnx, mtiles, ntiles_n, tile_m, tile_n);
        if (tile_m >= mtiles || tile_n >= ntiles_n) tile_m = -1;
        row_tile(tile_m, grouped, s_off, E, R, BM, mt);
    }
}

// Host side of map_tile: the order to use and the number of linear ids it spans.
// small_experts: a grouped launch whose experts hold a few row tiles each on average.
inline int pick_gnx(int ntiles_n, bool grouped = false, bool small_experts = false)
{
    // XCD-grouped orders only when the n-tiles split evenly over the XCDs (else XCDs idle)
    int gnx = ntiles_n % 8 == 0 ? 8 : 16;
    if (grouped && small_experts) gnx = 32;
    if (option(kOptGnx) >= 0) gnx = option(kOptGnx);   // tuning knob
    if (gnx == 32 && !grouped) gnx = ntiles_n % 8 == 0 ? 8 : 16;
    if (gnx != 0 && gnx != 4 && gnx != 8 && gnx != 16 && gnx != 32) gnx = 0;
    if (gnx == 4 && ntiles_n % 16 != 0) gnx = 0;
    if (gnx == 8 && ntiles_n % 8 != 0) gnx = 0;
    return gnx;
}
inline int64_t linear_ids(int gnx, int ntiles_m, int ntiles_n)
{
    if (gnx == 8) return static_cast<int64_t>(ntiles_n) * ntiles_m;     // exactly the tiles
    if (gnx == 16) return 8 * ceil_div(ntiles_m, 8) * ntiles_n;          // every XCD as long as the longest
    if (gnx == 32) return 8 * ceil_div(static_cast<int64_t>(ntiles_n) * ntiles_m, 8);
    if (gnx == 4) return ceil_div(ntiles_n, 16) * ceil_div(ntiles_m, 16) * 256;
    return static_cast<int64_t>(ntiles_n) * ntiles_m;
}

// Writes a wave's accumulators.  acc[j][i][v] is output row (X row) i*16 + lane%16 and output
// column j*16 + (lane/16)*4 + v of the WTM x WTN wave tile: four consecutive columns per lane,
// stored as one 8-byte word.  With SWIGLU sub-tiles j and j + TNS/2 hold gate and up columns.
template <typename T, int WTM, int WTN, bool SWIGLU>
__device__ __forceinline__ void tile_epilogue(float4_t (&acc)[WTN / 16][WTM / 16], const T *__restrict__ Bias,
                                              T *__restrict__ Y, const MTile &mt, int64_t N, int64_t ncols,
                                              int64_t n0, int wm, int wn, int lane)
{
    constexpr int TMS = WTM / 16, TNS = WTN / 16;
    const int lrow = lane & 15, lk = lane >> 4;
    const T *be = Bias ? Bias + static_cast<int64_t>(mt.e) * N : nullptr;
    const bool vec_ok = (ncols % 4 == 0) && (reinterpret_cast<uintptr_t>(Y) % 8 == 0);
#pragma unroll
    for (int i = 0; i < TMS; ++i) {
        const int row = wm * WTM + i * 16 + lrow;
        if (row >= mt.rows) continue;
        T *yrow = Y + (mt.row0 + row) * ncols;
#pragma unroll
        for (int j = 0; j < (SWIGLU ? TNS / 2 : TNS); ++j) {
            const int64_t n = (SWIGLU ? n0 + wn * (WTN / 2) : n0 + wn * WTN) + j * 16 + lk * 4;
            if (n >= ncols) continue;
            float val[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t nn = n + v < ncols ? n + v : ncols - 1;
                float g = acc[j][i][v] + (be ? to_f32(be[nn]) : 0.0f);
                if (SWIGLU) {
                    const float up = acc[j + TNS / 2][i][v] + (be ? to_f32(be[ncols + nn]) : 0.0f);
                    g = up * g * sigmoid_fast_(g);
                }
                val[v] = g;
            }
            if (vec_ok && n + 3 < ncols) {
                T out[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) out[v] = from_f32<T>(val[v]);
                *reinterpret_cast<uint2 *>(yrow + n) = *reinterpret_cast<const uint2 *>(out);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < ncols) yrow[n + v] = from_f32<T>(val[v]);
            }
        }
    }
}

// Same result as tile_epilogue, but staged through a wave-private LDS region (WTM rows of the
// wave's output columns, 16-byte chunks XOR-swizzled by row) so that global memory sees whole
// rows of the wave tile: each store instruction writes 1 KiB as runs of 128/256 contiguous
// bytes instead of 32-byte pieces.  No block barrier is needed (a wave only touches its own
// region, and its LDS operations execute in order); the caller guarantees that no wave still
// reads operand tiles from LDS.  Requires ncols % 8 == 0 and a 16-byte aligned Y.
//
// Everything that does not depend on the sub-tile row i is computed once per lane: the bias of
// the lane's columns, and the swizzled LDS addresses (a staged row is at most 16 chunks and
// sub-tiles start at multiples of 16 rows, so row % chunks == (lane % 16) % chunks for every
// i and the row part of the address is an instruction offset).
template <typename T, int WTM, int WTN, bool SWIGLU, bool BIAS>
__device__ __forceinline__ void tile_epilogue_lds_impl(float4_t (&acc)[WTN / 16][WTM / 16], const T *__restrict__ be,
                                                       T *__restrict__ Y, const MTile &mt, int64_t ncols, int64_t nw0,
                                                       int wm, int lane, char *wave_lds)
{
    constexpr int TMS = WTM / 16, TNS = WTN / 16, NO = SWIGLU ? TNS / 2 : TNS;
    constexpr int ROWP = NO * 16 * 2;          // bytes per staged row
    constexpr int CH16 = ROWP / 16;            // 16-byte chunks per staged row
    constexpr int RPI = 1024 / ROWP;           // rows per wave-wide 16-byte access
    static_assert(16 % CH16 == 0, "a staged row must hold 2, 4, 8 or 16 chunks");
    const int lrow = lane & 15, lk = lane >> 4;

    float bg[BIAS ? NO : 1][4], bu[BIAS && SWIGLU ? NO : 1][4];
    if (BIAS) {
#pragma unroll
        for (int j = 0; j < NO; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t n = nw0 + j * 16 + lk * 4 + v;
                const int64_t nn = n < ncols ? n : ncols - 1;
                bg[j][v] = to_f32(be[nn]);
                if (SWIGLU) bu[j][v] = to_f32(be[ncols + nn]);
            }
    }

    // chunk j*2 + lk/2 of row lrow (+ i*16) lands in slot chunk ^ (lrow % CH16)
    char *wbase = wave_lds + lrow * ROWP + (lk & 1) * 8;
    const int c0 = ((lk >> 1) ^ (lrow % CH16)) << 4;
#pragma unroll
    for (int i = 0; i < TMS; ++i) {
#pragma unroll
        for (int j = 0; j < NO; ++j) {
            T out[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float g = acc[j][i][v];
                if (BIAS) g += bg[j][v];
                if (SWIGLU) {
                    float up = acc[j + TNS / 2][i][v];
                    if (BIAS) up += bu[j][v];
                    g = up * g * sigmoid_fast_(g);
                }
                out[v] = from_f32<T>(g);
            }
            *reinterpret_cast<uint2 *>(wbase + (c0 ^ (j * 32)) + i * 16 * ROWP) = *reinterpret_cast<const uint2 *>(out);
        }
    }

    // read back whole rows: lane reads chunk c of row rr*RPI + lane/CH16
    const int c = lane % CH16, r0 = lane / CH16;
    const int64_t n = nw0 + c * 8;
    const bool col_ok = n < ncols;             // ncols % 8 == 0: a chunk is inside or outside as a whole
    T *yp = Y + (mt.row0 + wm * WTM + r0) * ncols + n;
    const int rows_left = static_cast<int>(mt.rows) - wm * WTM - r0;   // row rr*RPI is stored iff rr*RPI < rows_left
    constexpr int NR = WTM / RPI, BATCH = NR < 8 ? NR : 8;   // LDS reads in flight before their stores
#pragma unroll
    for (int r8 = 0; r8 < NR; r8 += BATCH) {
        u32x4 v[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int row = (r8 + u) * RPI + r0;   // row % CH16 takes CH16 / RPI (1 or 4) distinct per-lane values
            v[u] = *reinterpret_cast<const u32x4 *>(wave_lds + row * ROWP + ((c ^ (row % CH16)) << 4));
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            if (col_ok && (r8 + u) * RPI < rows_left) *reinterpret_cast<u32x4 *>(yp) = v[u];
            yp += static_cast<int64_t>(RPI) * ncols;
        }
    }
}

template <typename T, int WTM, int WTN, bool SWIGLU>
__device__ __forceinline__ void tile_epilogue_lds(float4_t (&acc)[WTN / 16][WTM / 16], const T *__restrict__ Bias,
                                                  T *__restrict__ Y, const MTile &mt, int64_t N, int64_t ncols,
                                                  int64_t n0, int wm, int wn, int lane, char *wave_lds)
{
    const int64_t nw0 = (SWIGLU ? n0 + wn * (WTN / 2) : n0 + wn * WTN);   // first output column of this wave
    if (Bias)
        tile_epilogue_lds_impl<T, WTM, WTN, SWIGLU, true>(acc, Bias + static_cast<int64_t>(mt.e) * N, Y, mt, ncols, nw0,
                                                          wm, lane, wave_lds);
    else
        tile_epilogue_lds_impl<T, WTM, WTN, SWIGLU, false>(acc, nullptr, Y, mt, ncols, nw0, wm, lane, wave_lds);
}

// Register-staged kernel: two LDS buffers, ONE register set staging global -> LDS, one barrier
// per k-tile.  A k-tile is four MFMA groups (K32 step 0/1 x lower/upper half of the wave's X
// rows); each group prefetches the fragments of the next one and carries its share of the
// LDS stores / global loads, the order inside a group pinned with sched_group_barrier.
template <typename T, int BM, int BN, int WM, int WN, bool SWIGLU>
__global__ __launch_bounds__(WM *WN * 64) void gemm_tiled_kernel(const T *__restrict__ X,
                                                                  const int64_t *__restrict__ off,
                                                                  const T *__restrict__ W,
                                                                  const T *__restrict__ Bias, int E, int64_t R,
                                                                  int64_t K, int64_t N, T *__restrict__ Y,
                                                                  int ntiles_n, int gnx,
                                                                  const int32_t *__restrict__ rt, int64_t xrows)
{
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;          // wave tile: WTM X-rows x WTN W-rows
    constexpr int TMS = WTM / 16, TNS = WTN / 16;        // 16x16 sub-tiles per wave
    constexpr int HM = TMS / 2;                          // X sub-tiles per MFMA group
    constexpr int BNO = SWIGLU ? BN / 2 : BN;            // output columns per tile
    constexpr int LA = BM * CH / NT, LB = BN * CH / NT;  // 16-byte loads per thread per k-tile
    constexpr int RSTEP = NT / CH;                       // tile rows between a thread's consecutive loads
    constexpr int STAGE = (BM + BN) * ROWB;
    static_assert(BM * CH % NT == 0 && BN * CH % NT == 0, "tile/threads mismatch");
    static_assert(TMS % 2 == 0 && RSTEP % 16 == 0, "wave tile too small");
    static_assert(!SWIGLU || TNS % 2 == 0, "SwiGLU needs an even number of n sub-tiles per wave");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ ExpertTable s_off;

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);

    stage_offsets(off, E, R, BM, s_off);
    MTile mt;
    int tile_n;
    locate_any(blockIdx.x, gnx, count_mtiles(off != nullptr, s_off, E, R, BM), ntiles_n, off != nullptr, s_off, E, R,
               BM, mt, tile_n);
    if (mt.rows == 0) return;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int64_t n0 = static_cast<int64_t>(tile_n) * BNO;
    const T *Xt = rt ? X : X + mt.row0 * K;      // with a row index (RowGather) offsets count from X itself
    const T *We = W + static_cast<int64_t>(mt.e) * N * K;

    // Staging: load q of a thread covers tile row tid/8 + RSTEP*q, 16-byte chunk tid%8.
    // RSTEP is a multiple of 16, so the swizzle term is the same for all of them and the
    // LDS destinations differ by compile-time constants.
    uint32_t a_src[LA], b_src[LB];   // byte offsets from the (uniform) tile base: scalar base + 32-bit lane offset loads
    const int srow = tid / CH, sc = tid % CH;
    const int dst0 = lds_off(srow, sc);
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = srow + RSTEP * i;
        const int r = row < mt.rows ? row : mt.rows - 1;
        a_src[i] = static_cast<uint32_t>(((rt ? gathered_row(rt, xrows, mt.row0 + r) : r) * K + sc * 8) * 2);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = srow + RSTEP * i;
        int64_t wrow;
        if (SWIGLU) {      // wave w's rows: WTN/2 gate rows, then the WTN/2 matching up rows
            const int w = row / WTN, jj = row % WTN, half = jj / (WTN / 2);
            int64_t ii = n0 + w * (WTN / 2) + jj % (WTN / 2);
            ii = ii < ncols ? ii : ncols - 1;
            wrow = half * ncols + ii;
        } else {
            wrow = n0 + row < N ? n0 + row : N - 1;
        }
        b_src[i] = static_cast<uint32_t>((wrow * K + sc * 8) * 2);
    }

    float4_t acc[TNS][TMS];
#pragma unroll
    for (int j = 0; j < TNS; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.0f;

    // Pipeline over k-tiles (tile kt sits in LDS buffer kt&1).  Group g = 2*s + h of a
    // k-tile multiplies the K32 step s of the W fragments wf[s] with X fragments xf[h]
    // (half h of the wave's X sub-tiles), after prefetching the fragments of group g+1:
    //   g+1 odd : xf[1] <- upper X half of the same step
    //   g+1 even: xf[0] <- lower X half and wf[s^1] <- W fragments of the next step.
    // Groups 0..2 also store their share of the staging registers (tile kt+1, loaded one
    // iteration ago) into buffer (kt+1)&1 and reload them with tile kt+2.  The barrier sits
    // before group 3, whose prefetch already reads tile kt+1.
    constexpr int KS = 4, NQ = LA + LB, QPK = (NQ + KS - 2) / (KS - 1), NM = HM * TNS;
    u32x4 rq[NQ];
    frag xf[2][HM], wf[2][TNS];
    const int nk = static_cast<int>(K / BK);
    const int lrow = lane & 15, lk = lane >> 4;
    const int swz = (lrow >> 1) & 7;                 // fragment rows differ from lrow by multiples of 16
    const int x_off = (wm * WTM + lrow) * ROWB;
    const int w_off = BM * ROWB + (wn * WTN + lrow) * ROWB;
    const int co0 = ((lk ^ swz) << 4), co1 = (((4 + lk) ^ swz) << 4);

#define OPMX_LOADQ(Q, KT)                                                                          \
    do {                                                                                           \
        const int64_t ko_ = static_cast<int64_t>(KT) * BK;                                         \
        if ((Q) < LA)                                                                              \
            rq[Q] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(Xt + ko_) +    \
                                                     a_src[(Q) < LA ? (Q) : 0]);                   \
        else                                                                                       \
            rq[Q] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(We + ko_) +    \
                                                     b_src[(Q) < LA ? 0 : (Q)-LA]);                \
    } while (0)
#define OPMX_DRAINQ(Q, BUF)                                                                        \
    do {                                                                                           \
        char *dst_ = smem + (BUF)*STAGE + dst0;                                                    \
        if ((Q) < LA) *reinterpret_cast<u32x4 *>(dst_ + (Q)*RSTEP * ROWB) = rq[Q];                 \
        else *reinterpret_cast<u32x4 *>(dst_ + BM * ROWB + ((Q)-LA) * RSTEP * ROWB) = rq[Q];       \
    } while (0)
    // fragments of group G of the tile in buffer BUF
#define OPMX_FRAGS(BUF, G)                                                                         \
    do {                                                                                           \
        const char *src_ = smem + (BUF)*STAGE + (((G) >> 1) ? co1 : co0);                          \
        if (((G)&1) == 0) {                                                                        \
            _Pragma("unroll") for (int i = 0; i < HM; ++i)                                         \
                xf[0][i] = *reinterpret_cast<const frag *>(src_ + x_off + i * 16 * ROWB);          \
            _Pragma("unroll") for (int j = 0; j < TNS; ++j)                                        \
                wf[((G) >> 1) & 1][j] = *reinterpret_cast<const frag *>(src_ + w_off + j * 16 * ROWB); \
        } else {                                                                                   \
            _Pragma("unroll") for (int i = 0; i < HM; ++i)                                         \
                xf[1][i] = *reinterpret_cast<const frag *>(src_ + x_off + (HM + i) * 16 * ROWB);   \
        }                                                                                          \
    } while (0)
#define OPMX_MMA(G)                                                                                \
    do {                                                                                           \
        _Pragma("unroll") for (int i = 0; i < HM; ++i)                                             \
            _Pragma("unroll") for (int j = 0; j < TNS; ++j)                                        \
                acc[j][((G)&1) * HM + i] =                                                         \
                    Mfma<T>::m16(wf[((G) >> 1) & 1][j], xf[(G)&1][i], acc[j][((G)&1) * HM + i]);   \
    } while (0)
    // Pin the order inside a group: one fragment read behind each of the first MFMAs, then
    // one LDS-store / global-load pair behind each of the following ones.
#define OPMX_ORDER(NREAD, NPAIR, DRAIN, LOAD)                                                      \
    do {                                                                                           \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                           \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                     \
            if (m < (NREAD)) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                    \
            const int p0 = (NREAD) < NM - (NPAIR) ? (NREAD) : (NM - (NPAIR) > 0 ? NM - (NPAIR) : 0); \
            if (m >= p0 && m < p0 + (NPAIR)) {                                                     \
                if (DRAIN) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                      \
                if (LOAD) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                       \
            }                                                                                      \
        }                                                                                          \
    } while (0)
#define OPMX_ITER(KT, DRAIN, LOAD, NEXT)                                                           \
    do {                                                                                           \
        _Pragma("unroll") for (int g = 0; g < KS - 1; ++g) {                                       \
            OPMX_FRAGS((KT)&1, g + 1);                                                             \
            OPMX_MMA(g);                                                                           \
            _Pragma("unroll") for (int qq = 0; qq < QPK; ++qq) {                                   \
                const int q = g * QPK + qq;                                                        \
                if (q < NQ) {                                                                      \
                    if (DRAIN) OPMX_DRAINQ(q, ((KT) + 1) & 1);                                     \
                    if (LOAD) OPMX_LOADQ(q, (KT) + 2);                                             \
                }                                                                                  \
            }                                                                                      \
            OPMX_ORDER(((g + 1) & 1) ? HM : HM + TNS,                                              \
                       (NQ - g * QPK < QPK ? (NQ - g * QPK > 0 ? NQ - g * QPK : 0) : QPK), DRAIN, LOAD); \
            __builtin_amdgcn_sched_barrier(0);                                                     \
        }                                                                                          \
        __syncthreads();                                                                           \
        if (NEXT) OPMX_FRAGS(((KT) + 1) & 1, 0);                                                   \
        OPMX_MMA(KS - 1);                                                                          \
        if (NEXT) OPMX_ORDER(HM + TNS, 0, false, false);                                           \
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
    OPMX_FRAGS(0, 0);
    {
        int kt = 0;
        for (; kt + 2 < nk; ++kt) OPMX_ITER(kt, true, true, true);
        if (kt + 1 < nk) {
            OPMX_ITER(kt, true, false, true);
            ++kt;
        }
        OPMX_ITER(kt, false, false, false);
    }
#undef OPMX_ITER
#undef OPMX_ORDER
#undef OPMX_MMA
#undef OPMX_FRAGS
#undef OPMX_DRAINQ
#undef OPMX_LOADQ

    // every wave passed the last barrier with its final fragments in registers: LDS is free
    if (ncols % 8 == 0 && reinterpret_cast<uintptr_t>(Y) % 16 == 0)
        tile_epilogue_lds<T, WTM, WTN, SWIGLU>(acc, Bias, Y, mt, N, ncols, n0, wm, wn, lane,
                                               smem + wave * (WTM * (SWIGLU ? WTN / 2 : WTN) * 2));
    else
        tile_epilogue<T, WTM, WTN, SWIGLU>(acc, Bias, Y, mt, N, ncols, n0, wm, wn, lane);
}

// ---------------------------------------------------------------------------------------
// Pieces of the direct-to-LDS kernel below.
#define OPMX_LPTR(p) ((void __attribute__((address_space(3))) *)(p))

// Block barrier WITHOUT a memory fence (a fence would wait for every in-flight direct-to-LDS
// load).  The caller orders explicitly: s_waitcnt vmcnt(0) for the tile it publishes,
// lgkmcnt(0) here for its own LDS reads of the buffer being retired.
__device__ __forceinline__ void barrier_no_fence()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Where the LDS fragment reads and the global -> LDS loads of a k-tile step sit among its four
// groups of MFMAs (OPMX_ITERX below).  `wide`: the wave tile has 8 column sub-tiles (128 x 128,
// 32 MFMAs per group, 16 loads per step) or 4 (128 x 64, 16 MFMAs per group, 12 loads per step).
__device__ __forceinline__ constexpr bool g0_reads(bool wide, int m) { return wide ? m % 2 == 0 : m < 12; }   // group 0: a read behind MFMA m?
__device__ __forceinline__ constexpr int g0_slot(bool wide, int m) { return wide ? m / 2 : m; }               // ... which of the 8 + TNS reads
__device__ __forceinline__ constexpr int g1_barrier(bool wide) { return wide ? 10 : 5; }                       // group 1: "buffer free" barrier
__device__ __forceinline__ constexpr int g1_load(bool wide, int m)                                             // group 1: load behind MFMA m, or -1
{
    return wide ? ((m >= 11 && (m - 11) % 3 == 0) ? (m - 11) / 3 : -1) : ((m >= 6 && m % 2 == 0) ? (m - 6) / 2 : -1);
}
__device__ __forceinline__ constexpr int g2_load(bool wide, int m)                                             // group 2: the remaining loads
{
    return wide ? ((m % 3 == 0 && m / 3 < 9) ? 7 + m / 3 : -1) : ((m % 2 == 0 && m / 2 < 7) ? 5 + m / 2 : -1);
}

// Waits until at most N vector-memory operations of this wave are outstanding (they complete
// in issue order, loads and stores alike).
template <int N> __device__ __forceinline__ void wait_vm()
{
    static_assert(N == 0 || N == 12 || N == 16 || N == 20 || N == 28 || N == 32 || N == 48, "add the immediate here");
    if (N == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (N == 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    if (N == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    if (N == 20) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
    if (N == 28) asm volatile("s_waitcnt vmcnt(28)" ::: "memory");
    if (N == 32) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
    if (N == 48) asm volatile("s_waitcnt vmcnt(48)" ::: "memory");
}

// Raw buffer descriptor over [base, base + 4 GiB): loads through it take a scalar base, a
// scalar offset and a 32-bit lane offset.
// `base` must be the same in every lane: it is forced into scalar registers, because a
// descriptor the compiler cannot prove uniform turns every load into a loop over lanes.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_descriptor(const void *base)
{
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((static_cast<uint64_t>(hi) << 32) | lo), 0,
                                             static_cast<int>(0xFFFFFFFFu), 0x00020000);
}

// Descriptor over `bytes` bytes from `base` (both uniform): accesses at offsets >= bytes are
// dropped by the hardware range check.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t bounded_descriptor(const void *base, uint32_t bytes)
{
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((static_cast<uint64_t>(hi) << 32) | lo), 0,
                                             static_cast<int>(__builtin_amdgcn_readfirstlane(bytes)), 0x00020000);
}

// 16 bytes per lane from descriptor + soff + voff straight into LDS at lds + 16*lane (lds is
// wave-uniform).
__device__ __forceinline__ void load_to_lds_16(__amdgpu_buffer_rsrc_t r, char *lds, uint32_t voff, int soff)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, OPMX_LPTR(lds), 16, voff, soff, 0, 0);
}

constexpr uint32_t kPastEveryX = 0x80000000u;   // a byte offset no gathered X reaches (x_descriptor)

// This lane's share of the sixteen 1 KiB wave loads per operand and k-tile: load i of wave w
// fetches tile rows 8*(w*L+i) .. +7, lane l the 16-byte chunk of row 8*(w*L+i) + l/8 that
// belongs in LDS slot l%8 of that row (slots are XOR-swizzled by row).  Results are byte offsets
// from the tile's X rows / the expert's W at k = 0.  W rows past the matrix repeat the last valid
// row (they feed accumulators that are never stored).  X rows past the tile keep their own
// offset: the tile's descriptor ends with its last row (x_descriptor), so the range check
// answers those loads with zeros -- the MFMAs of a ragged tile's missing rows then multiply
// zeros, which costs far less power than multiplying a copy of real data, and the part runs its
// MFMA kernels against a power limit.  With SWIGLU a wave's WTN W-rows are WTN/2 gate rows
// followed by the WTN/2 up rows of the same output columns.
template <int LA, int LB, int WTN, bool SWIGLU>
__device__ __forceinline__ void tile_sources(int rows, bool gather, int tokv, int64_t xrows, int64_t n0, int64_t K,
                                             int64_t N, int64_t ncols, int wave, int lane, uint32_t (&a_src)[LA],
                                             uint32_t (&b_src)[LB])
{
    const int lrow8 = lane >> 3, slot = lane & 7;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        const int row = (wave * LA + i) * 8 + lrow8;
        const int c = slot ^ ((row >> 1) & 7);
        if (!gather) {
            a_src[i] = static_cast<uint32_t>((row * K + c * 8) * 2);
        } else {
            // Through the row index (RowGather): offsets count from X itself.  Lane l of the wave
            // holds the index of the wave's l-th row (wave_row_index); each lane fetches the one of
            // its row by a cross-lane read and clamps it into X, like gathered_row(): a corrupt index
            // reads some row of X, never past it.  Rows the tile lacks get an offset past every X.
            const int raw = __shfl(tokv, i * 8 + lrow8, 64), last = static_cast<int>(xrows) - 1;
            const int tok = raw < 0 ? 0 : (raw > last ? last : raw);
            a_src[i] = row < rows ? static_cast<uint32_t>((static_cast<int64_t>(tok) * K + c * 8) * 2) : kPastEveryX;
        }
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
        const int row = (wave * LB + i) * 8 + lrow8;
        int64_t wrow;
        if (SWIGLU) {
            const int w = row / WTN, jj = row % WTN, half = jj / (WTN / 2);
            int64_t ii = n0 + w * (WTN / 2) + jj % (WTN / 2);
            ii = ii < ncols ? ii : ncols - 1;
            wrow = half * ncols + ii;
        } else {
            wrow = n0 + row < N ? n0 + row : N - 1;
        }
        const int c = slot ^ ((row >> 1) & 7);
        b_src[i] = static_cast<uint32_t>((wrow * K + c * 8) * 2);
    }
}

// Row index (RowGather) of the l-th X row that wave `wave` loads for the tile starting at row0
// (a wave loads RW = BM / 4 consecutive tile rows), in lane l; 0 without an index.  One load per
// lane, issued well ahead of tile_sources, which reads it across lanes and clamps it into X (the
// value is left as loaded here: arithmetic on it would wait for the load here).
template <int RW>
__device__ __forceinline__ int wave_row_index(const int32_t *__restrict__ rt, int64_t row0, int64_t R, int wave, int lane)
{
    if (rt == nullptr) return 0;
    const int64_t r = row0 + wave * RW + (lane < RW ? lane : RW - 1);
    return rt[r < R ? r : R - 1];
}

// Descriptor of a tile's X rows: `rows` rows of K elements from row `row0` on, and nothing behind
// them (loads of the rows a ragged tile lacks return zeros, see tile_sources).  With a row index
// (RowGather) it covers all xrows rows of X (xrows * K * 2 < 2^31) and tile_sources gives the
// lacking rows the offset kPastEveryX.
template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t x_descriptor(const T *X, int64_t row0, int rows, int64_t K,
                                                               const int32_t *rt, int64_t xrows)
{
    if (rt) return bounded_descriptor(X, static_cast<uint32_t>(xrows * K * 2));
    return bounded_descriptor(X + row0 * K, static_cast<uint32_t>(rows * K * 2));
}

// Where a workgroup starts its walk over the nk k-tiles (it wraps around): an eighth of K further
// on for every XCD.  The workgroups of one XCD keep walking together, which is what lets them
// share operand tiles in their L2, but the XCDs no longer ask the memory for the same k offset
// of every row at the same moment (rows lie a multiple of 8 KiB apart: such requests crowd onto
// few channels).  Down projection (K = 14336) +2.5 %, K = 4096 ... 6144 +0.6 ... 1 %; not worth it
// below 64 k-tiles.  The fp32 accumulation order then depends on the XCD, i.e. on the tile's
// position in the launch: fixed for a given problem shape.
__device__ __forceinline__ int k_rotation(int nk) { return nk >= 64 ? static_cast<int>(blockIdx.x & 7) * nk / 8 : 0; }

// Tail balancing ("split-K of the last round").  With G workgroup slots (one per CU) the last
// ttot % G tiles of the row-major tile order would run alone on a mostly idle chip.  When the
// caller lends scratch memory they are left to a second launch in which each of them is cut
// into `g` equal k-ranges, one workgroup each; the partial sums meet in the scratch memory.
// In the 2-D tile order (gnx = 4; the split is used with no other) the tile ids are exactly
// [0, ttot) and the tail ids are spread evenly over the XCDs; XCD j keeps the tail tiles it would
// have had (ids = j mod 8: a compact block of the tile grid) with all their k-ranges, so its
// workgroups walk the same k positions at the same time and keep sharing X- and W-tiles in L2.  g = 1: no split, the one-tile-per-workgroup launch does
// everything.  Must give the same answer on the host and on the device.
__host__ __device__ inline int sk_split(int64_t ttot, int sk_wgs, int nk, int gnx, int cost)
{
    if (sk_wgs < 8 || (gnx != 4 && gnx != 8)) return 1;
    const int64_t tail = ttot % sk_wgs;
    if (tail == 0) return 1;
    const int per_xcd = static_cast<int>((tail + 7) / 8);
    int g = (sk_wgs / 8) / per_xcd;
    if (g > nk / 8) g = nk / 8;          // at least 8 k-tiles per range
    if (g > 8) g = 8;
    if (g < 2) return 1;
    // the exchange of partial sums costs about as much as `cost` k-tiles of work; split only when
    // the time saved, (1 - 1/g) of a tile, is more
    return (g - 1) * nk > cost * g ? g : 1;
}

// ---------------------------------------------------------------------------------------
// Direct-to-LDS, 4 waves, fragments of a whole k-tile held in registers.  Each wave reads all
// 32 fragments of k-tile kt (128 VGPRs) by the first third of the k-tile, so the LDS buffer is
// free again a good k-tile before it is needed and the loads of k-tile kt+2 get more than a
// whole k-tile to land behind MFMAs: the slowest load of the slowest wave, which every wave
// waits for at the barrier, stops being the pace setter.  Two barriers per k-tile:
//   A (group 1, after this wave's last fragment read of buffer kt&1 returned): buffer free ->
//     16 loads of k-tile kt+2 into it, one every third MFMA of groups 1-2;
//   B (before group 3, after s_waitcnt vmcnt(16): this wave's loads of k-tile kt+1 landed) ->
//     group 3 reads the first fragments of k-tile kt+1.
// MFMAs are volatile asm (accumulators pinned to the 256 accumulation registers), so the
// source order below is the issue order.
// Partial sums cross XCDs (each has its own L2).  16-byte buffer accesses with the device-scope
// cache policy (sc0 sc1) write through to / read from the coherent level, which avoids the
// whole-L2 write-back and invalidate that a device-scope fence costs on this part; ordering
// against the arrival counter is by waiting for the stores (s_waitcnt vmcnt(0)) before the
// block barrier that precedes the counter update.  `slot` describes one fp32 tile-sized slot,
// `idx` counts 16-byte elements in it.
constexpr int kDeviceScope = 17;   // sc0 | sc1
__device__ __forceinline__ void coherent_store(__amdgpu_buffer_rsrc_t slot, int idx, float4_t v)
{
    u32x4 bits;
    __builtin_memcpy(&bits, &v, 16);
    __builtin_amdgcn_raw_buffer_store_b128(bits, slot, idx * 16, 0, kDeviceScope);
}
__device__ __forceinline__ float4_t coherent_load(__amdgpu_buffer_rsrc_t slot, int idx)
{
    const u32x4 bits = __builtin_amdgcn_raw_buffer_load_b128(slot, idx * 16, 0, kDeviceScope);
    float4_t v;
    __builtin_memcpy(&v, &bits, 16);
    return v;
}

// Scratch memory of the tail launch: arrival counters, then one fp32 tile-sized slot per workgroup.
constexpr int kSkCounters = 256;                  // tail tiles are fewer than the CUs
constexpr int kSkTile = 256 * 256;                // elements of an output tile

// The arrival counters of the tail tiles must read zero when the tail launch starts.  The first
// workgroup of the main launch clears them (count == nullptr: no tail launch follows): the tail
// launch is ordered behind the main one on the stream, and a kernel's writes are visible to the
// next kernel.  No memset and no launch of its own: callers may capture the sequence in a graph.
__device__ __forceinline__ void clear_tail_counters(int *__restrict__ count)
{
    if (count != nullptr && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kSkCounters; i += blockDim.x) count[i] = 0;
}

// SK = false: one tile per workgroup (all tiles, or all but the tail when sk_wgs > 0 and the
// tail is split).  SK = true: the tail launch, one k-range of one tail tile per workgroup.
template <typename T, int BM, int BN, bool SWIGLU, bool SK>
__global__ __launch_bounds__(256) void gemm_tiled_dlds_kernel(const T *__restrict__ X,
                                                               const int64_t *__restrict__ off,
                                                               const T *__restrict__ W,
                                                               const T *__restrict__ Bias, int E, int64_t R,
                                                               int64_t K, int64_t N, T *__restrict__ Y,
                                                               int ntiles_n, int gnx, int sk_wgs, int sk_cost,
                                                               float *__restrict__ sk_part, int *__restrict__ sk_count,
                                                               const int32_t *__restrict__ rt, int64_t xrows)
{
    constexpr int NW = 4, WM = BM / 128, WN = NW / WM;                 // 256 x 256: 2 x 2 waves, 128 x 256: 1 x 4
    constexpr int WTM = BM / WM, WTN = BN / WN, TMS = WTM / 16, TNS = WTN / 16, HM = TMS / 2;
    constexpr int BNO = SWIGLU ? BN / 2 : BN;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW, NL = LA + LB;   // 1 KiB wave loads per k-tile
    constexpr int STAGE = (BM + BN) * ROWB;
    constexpr int NM = HM * TNS;
    constexpr bool WIDE = TNS == 8;
    static_assert(HM == 4 && ((TNS == 8 && NL == 16) || (TNS == 4 && NL == 12)),
                  "the schedule below is written for 128x128 and 128x64 wave tiles");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];
    __shared__ ExpertTable s_off;

    __shared__ int s_arrivals;
    const int64_t ncols = SWIGLU ? N / 2 : N;
    if (!SK) zero_unowned_rows(Y, R, ncols, off, E);
    if (!SK) clear_tail_counters(sk_count);
    stage_offsets(off, E, R, BM, s_off);
    const int mtiles = count_mtiles(off != nullptr, s_off, E, R, BM);
    const int nk = static_cast<int>(K / BK);
    const int krot = k_rotation(nk);
    const int64_t ttot = static_cast<int64_t>(mtiles) * ntiles_n;
    const int g = sk_split(ttot, sk_wgs, nk, gnx, sk_cost);
    const int64_t tail = g > 1 ? ttot % sk_wgs : 0;      // tiles left to the tail launch
    MTile mt;
    int tile_n;
    int kt0 = 0, kt1 = nk;          // k-tiles of this workgroup
    int tail_tile = 0, chunk = 0;   // SK: which tail tile, which of its g k-ranges
    int xcd_first = 0, xcd_tiles = 0;
    if (!SK) {
        // with the orders the tail split is used with, the ids [0, ttot) are exactly the tiles,
        // and the last `tail` of them are spread evenly over the XCDs
        if (static_cast<int64_t>(blockIdx.x) >= ttot - tail && tail > 0) return;
        locate_any(blockIdx.x, gnx, mtiles, ntiles_n, off != nullptr, s_off, E, R, BM, mt, tile_n);
    } else {
        if (tail == 0) return;
        // XCD j (workgroups j, j+8, ...) takes the tail ids congruent to j mod 8 -- the tiles it
        // would have had in the other launch, a compact block of the tile grid -- with all their
        // k-ranges: position p = range * tiles + tile
        const int xcd = blockIdx.x & 7, p = blockIdx.x >> 3;
        const int64_t base = ttot - tail;
        xcd_first = static_cast<int>((xcd - base) & 7);                    // first tail tile of this XCD
        xcd_tiles = xcd_first < tail ? static_cast<int>((tail - xcd_first + 7) / 8) : 0;
        if (p >= xcd_tiles * g) return;
        chunk = p / xcd_tiles;
        tail_tile = xcd_first + 8 * (p % xcd_tiles);
        kt0 = chunk * nk / g;
        kt1 = (chunk + 1) * nk / g;
        locate_any(base + tail_tile, gnx, mtiles, ntiles_n, off != nullptr, s_off, E, R, BM, mt, tile_n);
    }
    if (mt.rows == 0) return;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int64_t n0 = static_cast<int64_t>(tile_n) * BNO;
    const __amdgpu_buffer_rsrc_t rx = x_descriptor(X, mt.row0, mt.rows, K, rt, xrows);
    const __amdgpu_buffer_rsrc_t rw = raw_descriptor(W + static_cast<int64_t>(mt.e) * N * K);

    uint32_t a_src[LA], b_src[LB];     // byte offsets from the tile's X / W base at k = 0
    tile_sources<LA, LB, WTN, SWIGLU>(mt.rows, rt != nullptr, wave_row_index<LA * 8>(rt, mt.row0, R, wave, lane), xrows, n0,
                                      K, N, ncols, wave, lane, a_src, b_src);
    const int a_lds = wave * LA * 1024, b_lds = BM * ROWB + wave * LB * 1024;   // wave-uniform

    float4_t acc[TNS][TMS];
#pragma unroll
    for (int j = 0; j < TNS; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.0f;

    const int lrow = lane & 15, lk = lane >> 4;
    const int swz = (lrow >> 1) & 7;
    const int x_off = (wm * WTM + lrow) * ROWB;
    const int w_off = BM * ROWB + (wn * WTN + lrow) * ROWB;
    const int co0 = ((lk ^ swz) << 4), co1 = (((4 + lk) ^ swz) << 4);
    frag xf[2][2][HM], wf[2][TNS];      // [k32 step][X half][sub-tile], [k32 step][sub-tile]

    // wave load Q of k-tile KT into buffer BUF: Q < LA -> X rows, else W rows
#define OPMX_ISSUE1(KT, BUF, Q)                                                                    \
    do {                                                                                           \
        char *st_ = smem + (BUF)*STAGE;                                                            \
        const int kr_ = (KT) + krot;                     /* rotated k-tile, see k_rotation */       \
        const int kb_ = (kr_ >= nk ? kr_ - nk : kr_) * ROWB;                                       \
        if ((Q) < LA) load_to_lds_16(rx, st_ + a_lds + (Q)*1024, a_src[(Q) < LA ? (Q) : 0], kb_);  \
        else load_to_lds_16(rw, st_ + b_lds + ((Q)-LA) * 1024, b_src[(Q) < LA ? 0 : (Q)-LA], kb_); \
    } while (0)
#define OPMX_XFRAG(BUF, S, H, I)                                                                   \
    xf[S][H][I] = *reinterpret_cast<const frag *>(smem + (BUF)*STAGE + ((S) ? co1 : co0) + x_off + ((H)*HM + (I)) * 16 * ROWB)
#define OPMX_WFRAG(BUF, S, J)                                                                      \
    wf[S][J] = *reinterpret_cast<const frag *>(smem + (BUF)*STAGE + ((S) ? co1 : co0) + w_off + (J)*16 * ROWB)
#define OPMX_MF(S, H, m) Mfma<T>::m16_acc(wf[S][(m) % TNS], xf[S][H][(m) / TNS], acc[(m) % TNS][(H)*HM + (m) / TNS])
    // the first k-tile of a tile overwrites the accumulators instead of adding to them
#define OPMX_MF0(FIRST, H, m)                                                                      \
    do {                                                                                           \
        if (FIRST) Mfma<T>::m16_first(wf[0][(m) % TNS], xf[0][H][(m) / TNS], acc[(m) % TNS][(H)*HM + (m) / TNS]); \
        else OPMX_MF(0, H, m);                                                                     \
    } while (0)
    // One k-tile, held in buffer B.  LD2: load k-tile LDK (of this tile: two k-tiles ahead; or one
    // of the first two of the workgroup's next tile) into buffer B once it is free, then wait
    // until at most VM vector-memory operations are outstanding; without LD2 wait for all.
    // NEXT: read the first fragments of the following k-tile from the other buffer.
#define OPMX_ITERX(LDK, B, LD2, NEXT, FIRST, VM)                                                   \
    do {                                                                                           \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                           \
            OPMX_MF0(FIRST, 0, m);                                                                 \
            if (g0_reads(WIDE, m)) {                                                               \
                const int r = g0_slot(WIDE, m);                                                    \
                if (r < 4) OPMX_XFRAG(B, 0, 1, r < 4 ? r : 0);                                     \
                else if (r < 8) OPMX_XFRAG(B, 1, 0, (r >= 4 && r < 8) ? r - 4 : 0);                \
                else OPMX_WFRAG(B, 1, (r >= 8 && r < 8 + TNS) ? r - 8 : 0);                        \
            }                                                                                      \
        }                                                                                          \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                           \
            OPMX_MF0(FIRST, 1, m);                                                                 \
            if (m < 4) OPMX_XFRAG(B, 1, 1, m < 4 ? m : 0);                                         \
            if (m == g1_barrier(WIDE)) barrier_no_fence();                                         \
            if ((LD2) && g1_load(WIDE, m) >= 0) OPMX_ISSUE1(LDK, B, g1_load(WIDE, m) >= 0 ? g1_load(WIDE, m) : 0); \
        }                                                                                          \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                           \
            OPMX_MF(1, 0, m);                                                                      \
            if ((LD2) && g2_load(WIDE, m) >= 0) OPMX_ISSUE1(LDK, B, g2_load(WIDE, m) >= 0 ? g2_load(WIDE, m) : 0); \
        }                                                                                          \
        wait_vm<(LD2) ? (VM) : 0>();                                                               \
        __builtin_amdgcn_s_barrier();                                                              \
        asm volatile("" ::: "memory");                                                             \
        _Pragma("unroll") for (int m = 0; m < NM; ++m) {                                           \
            OPMX_MF(1, 1, m);                                                                      \
            if ((NEXT) && m < 4) OPMX_XFRAG((B) ^ 1, 0, 0, m < 4 ? m : 0);                         \
            else if ((NEXT) && m < 4 + TNS) OPMX_WFRAG((B) ^ 1, 0, (m >= 4 && m < 4 + TNS) ? m - 4 : 0); \
        }                                                                                          \
    } while (0)
#define OPMX_ITER(KT, B, LD2, NEXT) OPMX_ITERX((KT) + 2, B, LD2, NEXT, false, NL)

    // prologue: first k-tile -> buffer 0, second -> buffer 1, wait for the first
#pragma unroll
    for (int q = 0; q < NL; ++q) OPMX_ISSUE1(kt0, 0, q);
    if (kt1 - kt0 > 1) {
#pragma unroll
        for (int q = 0; q < NL; ++q) OPMX_ISSUE1(kt0 + 1, 1, q);
        wait_vm<NL>();
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < HM; ++i) OPMX_XFRAG(0, 0, 0, i);
#pragma unroll
    for (int j = 0; j < TNS; ++j) OPMX_WFRAG(0, 0, j);
    {
        int kt = kt0, b = 0;
        for (; kt + 2 < kt1; ++kt, b ^= 1) OPMX_ITER(kt, b, true, true);
        if (kt + 1 < kt1) {
            OPMX_ITER(kt, b, false, true);
            ++kt;
            b ^= 1;
        }
        OPMX_ITER(kt, b, false, false);
    }
    // asm MFMAs are opaque to the compiler's hazard padding: let the last ones retire.  The
    // empty statements re-define every accumulator after the wait, so that whatever the register
    // allocator does with a finished accumulator (copy it out, spill it) is placed behind the
    // wait and not directly behind the MFMA that produced it, where it would read stale data.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int j = 0; j < TNS; ++j)
#pragma unroll
        for (int i = 0; i < TMS; ++i) asm volatile("" : "+a"(acc[j][i]));

    if (SK) {
        // A k-range of a tail tile.  Every workgroup parks its fp32 partial sums in its own slot
        // and adds its number of k-tiles to the tile's counter; the one that completes the count
        // adds all g partial sums up in k order (so the result does not depend on who was last)
        // and writes the tile.
        const __amdgpu_buffer_rsrc_t mine = raw_descriptor(sk_part + static_cast<int64_t>(blockIdx.x) * (BM * BN));
#pragma unroll
        for (int j = 0; j < TNS; ++j)
#pragma unroll
            for (int i = 0; i < TMS; ++i) coherent_store(mine, (j * TMS + i) * 256 + tid, acc[j][i]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0)
            s_arrivals = __hip_atomic_fetch_add(sk_count + tail_tile, kt1 - kt0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_arrivals + (kt1 - kt0) != nk) return;          // not the last one (uniform)
#pragma unroll
        for (int j = 0; j < TNS; ++j)
#pragma unroll
            for (int i = 0; i < TMS; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v) acc[j][i][v] = 0.0f;
        // the slot of k-range c of this tile: workgroup (this XCD, position c*tiles + tile)
        for (int c = 0; c < g; ++c) {
            const int wg = ((c * xcd_tiles + ((tail_tile - xcd_first) >> 3)) << 3) + (blockIdx.x & 7);
            const __amdgpu_buffer_rsrc_t theirs = raw_descriptor(sk_part + static_cast<int64_t>(wg) * (BM * BN));
            // sixteen loads in flight at a time: one at a time would be 64 serial round trips
#pragma unroll
            for (int blk = 0; blk < TNS * TMS / 16; ++blk) {
                float4_t part[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) part[u] = coherent_load(theirs, (blk * 16 + u) * 256 + tid);
#pragma unroll
                for (int u = 0; u < 16; ++u) acc[(blk * 16 + u) / TMS][(blk * 16 + u) % TMS] += part[u];
            }
        }
    }
    // after the last barrier no wave reads operand tiles any more: LDS is free for the epilogue
    if (ncols % 8 == 0 && reinterpret_cast<uintptr_t>(Y) % 16 == 0)
        tile_epilogue_lds<T, WTM, WTN, SWIGLU>(acc, Bias, Y, mt, N, ncols, n0, wm, wn, lane,
                                               smem + wave * (WTM * (SWIGLU ? WTN / 2 : WTN) * 2));
    else
        tile_epilogue<T, WTM, WTN, SWIGLU>(acc, Bias, Y, mt, N, ncols, n0, wm, wn, lane);
}

__device__ __forceinline__ void store_16(__amdgpu_buffer_rsrc_t r, uint32_t voff, u32x4 v)
{
    __builtin_amdgcn_raw_buffer_store_b128(v, r, voff, 0, 0);
}
constexpr uint32_t kDroppedStore = 0x80000000u;   // an offset past every tile (tiles are < 2 GiB)

// 8-byte LDS store the compiler does not see as one.  In front of a visible LDS store it waits
// for every outstanding direct-to-LDS load (it cannot tell that they land elsewhere), which in
// the persistent kernel are the next tile's first k-tiles, still in flight by design.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void lds_store_8_untracked(char *p, u32x2 v)
{
    const uint32_t a = (uint32_t)(size_t)OPMX_LPTR(p);
    asm volatile("ds_write_b64 %0, %1" ::"v"(a), "v"(v) : "memory");
}

// Epilogue of the persistent kernel.  Same values as tile_epilogue_lds, but
//  - staged through a small wave-private LDS region, 16 rows (one row of sub-tiles) at a time,
//    because the operand buffers already receive the next tile;
//  - stored through a descriptor over the tile's rows: lanes outside the tile (rows past its
//    end, columns past the matrix) get an offset the range check drops, so every wave issues
//    the same WTM * ROWP / 1024 stores whatever the tile's shape -- the caller's count of
//    outstanding memory operations depends on that;
//  - the stores of one pass are issued behind the LDS reads of the next.
// `ry` covers rows [row0, row0 + rows) of Y; requires ncols % 8 == 0 and a 16-byte aligned Y.
// The bias of this lane's output columns (gate columns in bg, up columns in bu), for
// tile_epilogue_staged_impl.  A function of its own so that the persistent kernel can issue
// these loads ahead of the last loads of a tile: waiting for them in the epilogue then leaves
// the younger loads of the next tile in flight.
template <typename T, int NO, bool SWIGLU>
__device__ __forceinline__ void load_bias_regs(const T *__restrict__ be, int64_t ncols, int64_t nw0, int lane,
                                               T (&bg)[NO][4], T (&bu)[NO][4])
{
    const int lk = lane >> 4;
#pragma unroll
    for (int j = 0; j < NO; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int64_t n = nw0 + j * 16 + lk * 4 + v;
            const int64_t nn = n < ncols ? n : ncols - 1;
            bg[j][v] = be[nn];             // left as loaded: converting here would wait for the load here
            bu[j][v] = be[SWIGLU ? ncols + nn : nn];
        }
}

template <typename T, int WTM, int WTN, bool SWIGLU, bool BIAS>
__device__ __forceinline__ void tile_epilogue_staged_impl(
    float4_t (&acc)[WTN / 16][WTM / 16], const T (&bg)[SWIGLU ? WTN / 32 : WTN / 16][4],
    const T (&bu)[SWIGLU ? WTN / 32 : WTN / 16][4], __amdgpu_buffer_rsrc_t ry, int64_t ncols, int64_t nw0, int wm,
    int lane, char *stg)
{
    constexpr int TMS = WTM / 16, TNS = WTN / 16, NO = SWIGLU ? TNS / 2 : TNS;
    constexpr int ROWP = NO * 16 * 2;          // bytes per staged row
    constexpr int CH16 = ROWP / 16;            // 16-byte chunks per staged row
    constexpr int RPI = 1024 / ROWP;           // rows per wave-wide 16-byte access
    constexpr int NRD = 16 / RPI;              // accesses per pass of 16 rows
    static_assert(16 % CH16 == 0 && 16 % RPI == 0, "staged row must hold 4, 8 or 16 chunks");
    const int lrow = lane & 15, lk = lane >> 4;
    char *wbase = stg + lrow * ROWP + (lk & 1) * 8;
    const int c0 = ((lk >> 1) ^ (lrow % CH16)) << 4;
    const int c = lane % CH16, r0 = lane / CH16;
    const int64_t n = nw0 + c * 8;
    // byte offset of (tile row wm*WTM + r0, column n); one pass further down is 16 rows
    uint32_t voff = n < ncols ? static_cast<uint32_t>(((wm * WTM + r0) * ncols + n) * 2) : kDroppedStore;
    const uint32_t row_bytes = static_cast<uint32_t>(ncols * 2);
    u32x4 held[NRD];
#pragma unroll
    for (int i = 0; i <= TMS; ++i) {
        // keep every pass's accumulator reads inside the pass: moved to the front they would need
        // a vector register each while the next tile's fragments and offsets are live
        __builtin_amdgcn_sched_barrier(0);
        u32x4 now[NRD];
        if (i < TMS) {
#pragma unroll
            for (int j = 0; j < NO; ++j) {
                T out[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float g = acc[j][i][v];
                    if (BIAS) g += to_f32(bg[j][v]);
                    if (SWIGLU) {
                        float up = acc[j + TNS / 2][i][v];
                        if (BIAS) up += to_f32(bu[j][v]);
                        g = up * g * sigmoid_fast_(g);
                    }
                    out[v] = from_f32<T>(g);
                }
                u32x2 bits;
                __builtin_memcpy(&bits, out, 8);
                lds_store_8_untracked(wbase + (c0 ^ (j * 32)), bits);
            }
#pragma unroll
            for (int u = 0; u < NRD; ++u) {
                const int row = u * RPI + r0;
                now[u] = *reinterpret_cast<const u32x4 *>(stg + row * ROWP + ((c ^ (row % CH16)) << 4));
            }
        }
        if (i > 0) {
#pragma unroll
            for (int u = 0; u < NRD; ++u) {
                // n >= ncols keeps the dropped offset: adding rows to it stays far past the tile
                store_16(ry, voff, held[u]);
                voff += (n < ncols ? RPI : 0) * row_bytes;
            }
        }
#pragma unroll
        for (int u = 0; u < NRD; ++u) held[u] = now[u];
    }
}

// Persistent form of gemm_tiled_dlds_kernel: one workgroup per CU walks the tile ids
// blockIdx.x, blockIdx.x + gridDim.x, ... (XCD-aware tile orders only, K >= 4 k-tiles) and treats them
// as one continuous stream of k-tiles.  The last two k-tile steps of a tile already load the
// first two k-tiles of the next one, so there is no pipeline refill between tiles, and the
// output stores of a tile drain behind the MFMAs of the next: they are issued after those loads,
// and vector-memory operations complete in issue order, so the first step of the next tile
// waits with a count that leaves the stores (a fixed number per wave, see
// tile_epilogue_staged_impl) and its own new loads outstanding.
// Covers the tile ids the tail launch does not take (see sk_split).
template <typename T, int BM, int BN, bool SWIGLU, bool BIAS>
__global__ __launch_bounds__(256) void gemm_tiled_dlds_persist_kernel(const T *__restrict__ X,
                                                                       const int64_t *__restrict__ off,
                                                                       const T *__restrict__ W,
                                                                       const T *__restrict__ Bias, int E, int64_t R,
                                                                       int64_t K, int64_t N, T *__restrict__ Y,
                                                                       int ntiles_n, int gnx, int sk_wgs, int sk_cost,
                                                                       int *__restrict__ sk_count,
                                                                       const int32_t *__restrict__ rt, int64_t xrows)
{
    constexpr int NW = 4, WM = BM / 128, WN = NW / WM;                 // 256 x 256: 2 x 2 waves, 128 x 256: 1 x 4
    constexpr int WTM = BM / WM, WTN = BN / WN, TMS = WTM / 16, TNS = WTN / 16, HM = TMS / 2;
    constexpr int BNO = SWIGLU ? BN / 2 : BN;
    constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW, NL = LA + LB;
    constexpr int STAGE = (BM + BN) * ROWB;
    constexpr int NM = HM * TNS;
    constexpr int STG = 16 * (SWIGLU ? WTN / 2 : WTN) * 2;            // staging bytes per wave: 16 output rows
    constexpr int NS = WTM * (SWIGLU ? WTN / 2 : WTN) * 2 / 1024;      // output stores per wave and tile
    static_assert(HM == 4 && ((TNS == 8 && NL == 16) || (TNS == 4 && NL == 12)),
                  "the schedule is written for 128x128 and 128x64 wave tiles");
    constexpr int NOB = SWIGLU ? TNS / 2 : TNS;                       // output sub-tile columns per wave
    constexpr bool WIDE = TNS == 8;
    static_assert(NS == 8 || NS == 16 || NS == 32, "wait counts below");
    using frag = typename Mfma<T>::frag;

    extern __shared__ __attribute__((aligned(16))) char smem[];      // two stages, then NW staging regions
    __shared__ ExpertTable s_off;

    const int64_t ncols = SWIGLU ? N / 2 : N;
    zero_unowned_rows(Y, R, ncols, off, E);
    clear_tail_counters(sk_count);
    stage_offsets(off, E, R, BM, s_off);
    const int mtiles = count_mtiles(off != nullptr, s_off, E, R, BM);
    const int nk = static_cast<int>(K / BK);
    const int krot = k_rotation(nk);
    const int64_t ttot = static_cast<int64_t>(mtiles) * ntiles_n;
    const int g = sk_split(ttot, sk_wgs, nk, gnx, sk_cost);
    // ids [nmain, ttot) are the tail launch's.  The row-partition order has ids that name no tile
    // behind the last tile of each XCD: its id space is longer than the tile count, and a
    // workgroup's stream ends at the first such id (all later ones of its XCD are empty too).
    const int64_t ids = gnx == 16 ? int64_t{8} * ((mtiles + 7) / 8) * ntiles_n : (gnx == 32 ? (ttot + 7) / 8 * 8 : ttot);
    const int64_t nmain = g > 1 ? ttot - ttot % sk_wgs : ids;
    int64_t id = blockIdx.x;
    if (id >= nmain) return;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    MTile cur;
    int cur_n;
    locate_any(id, gnx, mtiles, ntiles_n, off != nullptr, s_off, E, R, BM, cur, cur_n);
    if (cur.rows == 0) return;
    __amdgpu_buffer_rsrc_t rx = x_descriptor(X, cur.row0, cur.rows, K, rt, xrows);
    __amdgpu_buffer_rsrc_t rw = raw_descriptor(W + static_cast<int64_t>(cur.e) * N * K);
    uint32_t a_src[LA], b_src[LB];
    tile_sources<LA, LB, WTN, SWIGLU>(cur.rows, rt != nullptr, wave_row_index<LA * 8>(rt, cur.row0, R, wave, lane), xrows,
                                      static_cast<int64_t>(cur_n) * BNO, K, N, ncols, wave, lane, a_src, b_src);
    const int a_lds = wave * LA * 1024, b_lds = BM * ROWB + wave * LB * 1024;
    char *stg = smem + 2 * STAGE + wave * STG;

    float4_t acc[TNS][TMS];            // every tile's first k-tile defines all of them

    const int lrow = lane & 15, lk = lane >> 4;
    const int swz = (lrow >> 1) & 7;
    const int x_off = (wm * WTM + lrow) * ROWB;
    const int w_off = BM * ROWB + (wn * WTN + lrow) * ROWB;
    const int co0 = ((lk ^ swz) << 4), co1 = (((4 + lk) ^ swz) << 4);
    frag xf[2][2][HM], wf[2][TNS];

#pragma unroll
    for (int q = 0; q < NL; ++q) OPMX_ISSUE1(0, 0, q);
#pragma unroll
    for (int q = 0; q < NL; ++q) OPMX_ISSUE1(1, 1, q);
    wait_vm<NL>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < HM; ++i) OPMX_XFRAG(0, 0, 0, i);
#pragma unroll
    for (int j = 0; j < TNS; ++j) OPMX_WFRAG(0, 0, j);

    // The first step of a tile waits with a count that leaves the previous tile's NS stores
    // outstanding (below).  Give the first tile the same history: NS stores the range check drops.
    {
        const __amdgpu_buffer_rsrc_t nowhere = bounded_descriptor(Y, 0);
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < NS; ++u) store_16(nowhere, kDroppedStore + 16 * u, zero);   // distinct: none is redundant
    }

    int b = 0;
    for (;;) {
        // The workgroup's next tile (uniform).  Without one the last two steps load this tile's
        // first k-tiles again, into buffers nobody reads any more: one code path for the
        // accumulators, no matter whether a tile follows.
        const int64_t nid = id + gridDim.x;
        MTile nxt = cur;
        int nxt_n = cur_n;
        bool has_next = false;
        if (nid < nmain) {
            MTile t;
            locate_any(nid, gnx, mtiles, ntiles_n, off != nullptr, s_off, E, R, BM, t, nxt_n);
            has_next = t.rows > 0;
            if (has_next) nxt = t;
            else nxt_n = cur_n;
        }
        // the next tile's row indices (RowGather), requested a whole tile ahead of their use
        const int nxt_tok = wave_row_index<LA * 8>(rt, nxt.row0, R, wave, lane);

        // k-tile 0 overwrites the accumulators.  When k-tile 1 is known to have landed, the NS
        // stores of the previous tile and the NL loads of this step may still be outstanding.
        OPMX_ITERX(2, b, true, true, true, NL + NS);
        b ^= 1;
        for (int kt = 1; kt + 2 < nk; ++kt, b ^= 1) OPMX_ITERX(kt + 2, b, true, true, false, NL);
        // all loads of this tile are issued: retarget the load state, then stream on
        rx = x_descriptor(X, nxt.row0, nxt.rows, K, rt, xrows);
        rw = raw_descriptor(W + static_cast<int64_t>(nxt.e) * N * K);
        tile_sources<LA, LB, WTN, SWIGLU>(nxt.rows, rt != nullptr, nxt_tok, xrows, static_cast<int64_t>(nxt_n) * BNO, K, N, ncols,
                                          wave, lane, a_src, b_src);
        const int64_t nw0 = static_cast<int64_t>(cur_n) * BNO + wn * (SWIGLU ? WTN / 2 : WTN);   // first output column of this wave
        T bg[NOB][4], bu[NOB][4];          // bias of this lane's columns, requested ahead of the last loads
        if (BIAS) load_bias_regs<T, NOB, SWIGLU>(Bias + static_cast<int64_t>(cur.e) * N, ncols, nw0, lane, bg, bu);
        OPMX_ITERX(0, b, true, true, false, NL);
        b ^= 1;
        OPMX_ITERX(1, b, true, true, false, NL);
        b ^= 1;
        // let the last MFMAs retire; re-define the accumulators behind the wait (see
        // gemm_tiled_dlds_kernel)
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
        for (int j = 0; j < TNS; ++j)
#pragma unroll
            for (int i = 0; i < TMS; ++i) asm volatile("" : "+a"(acc[j][i]));

        {
            const __amdgpu_buffer_rsrc_t ry =
                bounded_descriptor(Y + cur.row0 * ncols, static_cast<uint32_t>(cur.rows * ncols * 2));
            // BIAS is a kernel parameter, not a branch: the bias instance needs registers for the
            // lane's bias values, and in one kernel the other path would pay for them with spills
            tile_epilogue_staged_impl<T, WTM, WTN, SWIGLU, BIAS>(acc, bg, bu, ry, ncols, nw0, wm, lane, stg);
        }
        if (!has_next) break;
        cur = nxt;
        cur_n = nxt_n;
        id = nid;
    }
    // the loads issued for a tile that does not follow must land before the LDS goes away
    wait_vm<0>();
}
#undef OPMX_ITER
#undef OPMX_ITERX
#undef OPMX_MF0
#undef OPMX_MF
#undef OPMX_WFRAG
#undef OPMX_XFRAG
#undef OPMX_ISSUE1

template <typename T, int BM, int BN, int WM, int WN>
int tiled_launch(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                   int64_t N, int epilogue, void *Y, hipStream_t s, RowGather g)
{
    constexpr int smem = 2 * (BM + BN) * ROWB;
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    const int64_t ncols = sw ? N / 2 : N;
    const int ntiles_n = static_cast<int>(ceil_div(ncols, sw ? BN / 2 : BN));
    const int ntiles_m = static_cast<int>(max_mtiles(R, E, BM));
    const int gnx = pick_gnx(ntiles_n);
    const int64_t nblocks = linear_ids(gnx, ntiles_m, ntiles_n);
    dim3 grid(static_cast<unsigned>(nblocks));
    dim3 block(WM * WN * 64);
    static std::atomic<uint64_t> attr_done[2];
    if (sw) {
        auto kern = gemm_tiled_kernel<T, BM, BN, WM, WN, true>;
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done[1])) return OPMX_ERR_LAUNCH;
        kern<<<grid, block, smem, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                       static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), ntiles_n, gnx, g.index,
                                       g.x_rows);
    } else {
        auto kern = gemm_tiled_kernel<T, BM, BN, WM, WN, false>;
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kern), smem, attr_done[0])) return OPMX_ERR_LAUNCH;
        kern<<<grid, block, smem, s>>>(static_cast<const T *>(X), off, static_cast<const T *>(W),
                                       static_cast<const T *>(B), E, R, K, N, static_cast<T *>(Y), ntiles_n, gnx, g.index,
                                       g.x_rows);
    }
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

// arrival counters, then one fp32 tile-sized slot per workgroup of the tail launch
size_t sk_workspace_bytes(int cus)
{
    return static_cast<size_t>(kSkCounters) * sizeof(int) + static_cast<size_t>(cus) * kSkTile * sizeof(float);
}

template <typename T, int BM, int BN>
int tiled_dlds_launch(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                      int64_t K, int64_t N, int epilogue, void *Y, void *ws, size_t ws_bytes, hipStream_t s, RowGather g)
{
    static_assert(BM * BN <= kSkTile, "tail slot size");
    constexpr int smem = 2 * (BM + BN) * ROWB;
    const bool sw = epilogue == OPMX_EPILOGUE_SWIGLU;
    const int64_t ncols = sw ? N / 2 : N;
    const int ntiles_n = static_cast<int>(ceil_div(ncols, sw ? BN / 2 : BN));
    const int ntiles_m = static_cast<int>(max_mtiles(R, E, BM));
    // Many small experts -- on average up to 96 tiles each, three times what an XCD holds at a time --
    // and no tail split: expert-grouped order.  Measured against the expert-major / row-partition
    // orders: 64 experts x (2-3 row tiles x 11 or 8 column tiles) -11 % and -12 % time, 4-5 row tiles
    // -3 % and -3 %, 8-9 row tiles +1 % and -5 %; 128 experts x (4-5 x 6 or 8) -5 % and -4 %; experts of
    // 170 tiles and more +6 ... +14 % (an XCD alone on an expert re-reads its X rows for every handful
    // of columns, and no other XCD has brought them into the memory-side cache).
    const bool small_experts = off != nullptr && K / BK <= 128 && (2 * R + int64_t{E} * BM) * ntiles_n <= int64_t{192} * E * BM;
    const int gnx = pick_gnx(ntiles_n, off != nullptr, small_experts);
    const int64_t dp_ids = linear_ids(gnx, ntiles_m, ntiles_n);
    if (dp_ids >= (int64_t{1} << 31)) return OPMX_ERR_UNSUPPORTED;
    // split-K of the tail tiles when the caller lends the scratch memory for it.  The tile count
    // is only known on the device, so the tail launch is always made; it exits at once when
    // there is no tail or no split.
    const int cus = cu_count();
    int sk_wgs = 0;
    if (ws != nullptr && cus >= 8 && cus % 8 == 0 && cus <= kSkCounters && ws_bytes >= sk_workspace_bytes(cus) &&
        reinterpret_cast<uintptr_t>(ws) % 16 == 0 && (gnx == 4 || gnx == 8))
        sk_wgs = cus;
    // Measured: the exchange costs ~100 us against 1.43 us per k-tile.
    int sk_cost = 70;
    if (option(kOptStreamK) == 0) sk_wgs = 0;    // tuning knob: 0 = off, 2 = split whenever possible
    if (option(kOptStreamK) == 2) sk_cost = 0;
    if (7 * (K / BK) <= 8 * sk_cost) sk_wgs = 0;     // sk_split() cannot split a K this short (g <= 8)
    int *sk_count = sk_wgs > 0 ? static_cast<int *>(ws) : nullptr;      // nullptr: no tail launch, nothing to clear
    float *sk_part = reinterpret_cast<float *>(static_cast<char *>(ws) + kSkCounters * sizeof(int));
    dim3 grid(static_cast<unsigned>(dp_ids));
    dim3 block(256);
    static std::atomic<uint64_t> attr_done[2][2];
    {
        const void *k1 = sw ? reinterpret_cast<const void *>(gemm_tiled_dlds_kernel<T, BM, BN, true, false>)
                            : reinterpret_cast<const void *>(gemm_tiled_dlds_kernel<T, BM, BN, false, false>);
        const void *k2 = sw ? reinterpret_cast<const void *>(gemm_tiled_dlds_kernel<T, BM, BN, true, true>)
                            : reinterpret_cast<const void *>(gemm_tiled_dlds_kernel<T, BM, BN, false, true>);
        if (!ensure_dynamic_smem(k1, smem, attr_done[sw ? 1 : 0][0]) || !ensure_dynamic_smem(k2, smem, attr_done[sw ? 1 : 0][1]))
            return OPMX_ERR_LAUNCH;
    }
    const T *Xp = static_cast<const T *>(X), *Wp = static_cast<const T *>(W), *Bp = static_cast<const T *>(B);
    T *Yp = static_cast<T *>(Y);
    // Persistent form (one workgroup per CU streams through its tiles) when its conditions hold
    // (2-D tile order, at least 4 k-tiles, whole 16-byte output chunks, tiles under 2 GiB) and K is
    // short enough for the tile switch to matter.  Measured: +3-12 % up to K = 4096, even at
    // 8192, -2 % at K = 14336, where the fixed pairing of workgroups and tiles lets the
    // workgroups of an XCD drift apart over the rounds and share less in L2 (+13 % HBM reads).
    bool persist = (gnx == 4 || gnx == 8 || gnx == 16 || gnx == 32) && K / BK >= 4 && ncols % 8 == 0 && reinterpret_cast<uintptr_t>(Y) % 16 == 0 &&
                   ncols * (2 * BM) < (int64_t{1} << 31) && cus >= 8 && cus % 8 == 0;
    if (option(kOptPersist) >= 0) {              // tuning knob: 0 = never, 1 = whenever possible
        if (option(kOptPersist) == 0) persist = false;
    } else if (K / BK > 128) {
        persist = false;
    }
    {
        // 128 x 256 tiles: the persistent form pays while a tile is short (its fixed cost of about
        // 8 us outside the k loop is then a tenth of the tile and more)
        if constexpr (BM == 128)
            if (option(kOptPersist) < 0 && K / BK > 128) persist = false;
    }
    if (persist) {
        constexpr int WTN_ = BN / (4 / (BM / 128));                          // columns of a wave tile
        const int smem_p = smem + 4 * 16 * (sw ? WTN_ / 2 : WTN_) * 2;       // + the four staging regions
        static std::atomic<uint64_t> attr_p[4];
        const bool hb = B != nullptr;
        using kernel_t = void (*)(const T *, const int64_t *, const T *, const T *, int, int64_t, int64_t, int64_t, T *, int,
                                  int, int, int, int *, const int32_t *, int64_t);
        const kernel_t kp = sw ? (hb ? gemm_tiled_dlds_persist_kernel<T, BM, BN, true, true>
                                     : gemm_tiled_dlds_persist_kernel<T, BM, BN, true, false>)
                               : (hb ? gemm_tiled_dlds_persist_kernel<T, BM, BN, false, true>
                                     : gemm_tiled_dlds_persist_kernel<T, BM, BN, false, false>);
        const int slot = (sw ? 2 : 0) + (hb ? 1 : 0);
        if (!ensure_dynamic_smem(reinterpret_cast<const void *>(kp), smem_p, attr_p[slot])) return OPMX_ERR_LAUNCH;
        // ids congruent mod 8 stay on one XCD as long as the grid is a multiple of 8
        const unsigned wgs = static_cast<unsigned>(dp_ids < cus ? dp_ids : cus);
        kp<<<wgs, block, smem_p, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n, gnx, sk_wgs, sk_cost, sk_count, g.index, g.x_rows);
        if (sk_wgs > 0) {
            if (sw)
                gemm_tiled_dlds_kernel<T, BM, BN, true, true><<<sk_wgs, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                          gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
            else
                gemm_tiled_dlds_kernel<T, BM, BN, false, true><<<sk_wgs, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                           gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
        }
        OPMX_LAUNCH_CHECK();
        return OPMX_OK;
    }
    if (sw) {
        gemm_tiled_dlds_kernel<T, BM, BN, true, false><<<grid, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                 gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
        if (sk_wgs > 0)
            gemm_tiled_dlds_kernel<T, BM, BN, true, true><<<sk_wgs, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                      gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
    } else {
        gemm_tiled_dlds_kernel<T, BM, BN, false, false><<<grid, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                  gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
        if (sk_wgs > 0)
            gemm_tiled_dlds_kernel<T, BM, BN, false, true><<<sk_wgs, block, smem, s>>>(Xp, off, Wp, Bp, E, R, K, N, Yp, ntiles_n,
                                                                                       gnx, sk_wgs, sk_cost, sk_part, sk_count, g.index, g.x_rows);
    }
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

template <typename T>
int tiled_impl(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
               int64_t N, int epilogue, int variant, void *Y, void *ws, size_t ws_bytes, hipStream_t s, RowGather g)
{
    switch (variant) {
        case 1: return tiled_launch<T, 256, 256, 2, 4>(X, off, W, B, E, R, K, N, epilogue, Y, s, g);
        case 2: return tiled_launch<T, 128, 128, 2, 2>(X, off, W, B, E, R, K, N, epilogue, Y, s, g);
        case 3: return tiled_dlds_launch<T, 128, 256>(X, off, W, B, E, R, K, N, epilogue, Y, ws, ws_bytes, s, g);
        default: return tiled_dlds_launch<T, 256, 256>(X, off, W, B, E, R, K, N, epilogue, Y, ws, ws_bytes, s, g);
    }
}

}  // namespace

// Requires: dtype f16/bf16, K % 64 == 0, 16-byte aligned X and W, N*K < 2^31.
// ws / ws_bytes: optional scratch memory (gemm_tiled_workspace_bytes()); with it the default
// variant balances the last rounds of tiles over all CUs.
int launch_gemm_tiled(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                      int64_t K, int64_t N, int dtype, int epilogue, int variant, void *Y, void *ws,
                      size_t ws_bytes, hipStream_t s, RowGather g)
{
    // offsets into a gathered X are 32 bits wide and kPastEveryX must lie behind it
    if (g.index != nullptr && g.x_rows * K * 2 >= (int64_t{1} << 31)) return OPMX_ERR_UNSUPPORTED;
    switch (dtype) {
        case OPMX_DTYPE_F16: return tiled_impl<f16>(X, off, W, B, E, R, K, N, epilogue, variant, Y, ws, ws_bytes, s, g);
        case OPMX_DTYPE_BF16: return tiled_impl<bf16>(X, off, W, B, E, R, K, N, epilogue, variant, Y, ws, ws_bytes, s, g);
    }
    return OPMX_ERR_UNSUPPORTED;
}

size_t gemm_tiled_workspace_bytes()
{
    const int cus = cu_count();
    return cus > 0 ? sk_workspace_bytes(cus) : 0;
}

}  // namespace opmx
