// Pieces shared by the grouped-GEMM kernels: the on-device tile scheduler that
// turns expert_offset into (expert, row range) work items without a host sync,
// MFMA fragment types and the zero-fill of rows no expert owns.
#pragma once
#include "common.h"

namespace opmx {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // a 16-byte register quad
typedef float float16_t __attribute__((ext_vector_type(16)));

template <typename T> struct Mfma;
template <> struct Mfma<f16> {
    using frag = half8_t;
    static __device__ __forceinline__ float16_t m32(frag a, frag b, float16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4_t m16(frag a, frag b, float4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    // Accumulate in place with the accumulator pinned to an accumulation register quad.
    // For kernels whose accumulators fill that register file completely: the builtin form
    // leaves destination and addend as separate values, and with no spare quad the register
    // allocator then shuffles accumulators through vector registers.  Volatile: keeps
    // source order against memory instructions, which is how those kernels pin their
    // MFMA / memory interleave.  The compiler inserts no hazard padding around it.
    static __device__ __forceinline__ void m16_acc(frag a, frag b, float4_t &c)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    // c = a*b (addend 0) into an accumulation register quad: starts a new accumulation without
    // clearing the accumulators, and without carrying their old values along (in a loop over
    // tiles that would make them loop-carried values the register allocator moves about).
    static __device__ __forceinline__ void m16_first(frag a, frag b, float4_t &c)
    {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }
};
template <> struct Mfma<bf16> {
    using frag = bf16x8_t;
    static __device__ __forceinline__ float16_t m32(frag a, frag b, float16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float4_t m16(frag a, frag b, float4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ void m16_acc(frag a, frag b, float4_t &c)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    // c = a*b (addend 0) into an accumulation register quad: starts a new accumulation without
    // clearing the accumulators, and without carrying their old values along (in a loop over
    // tiles that would make them loop-carried values the register allocator moves about).
    static __device__ __forceinline__ void m16_first(frag a, frag b, float4_t &c)
    {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }
};

// Rows of a grouped GEMM's X operand taken through an index instead of in place: GEMM row r is
// X[index[r], :] and X has x_rows rows (index == nullptr: row r is X[r, :]).  This is how the
// gate/up GEMM reads the tokens of MoeSelect's permuted order without X_expand_permute
// (MoeSelect.py:45-47) ever being written: index[r] = perm[r] / k.
struct RowGather {
    const int32_t *index = nullptr;
    int64_t x_rows = 0;
};
// The row of X that GEMM row r reads, clamped into X (a corrupt index cannot leave the tensor; the
// direct-to-LDS kernels clamp the same way where they turn the index into an offset).
__device__ __forceinline__ int64_t gathered_row(const int32_t *__restrict__ index, int64_t x_rows, int64_t r)
{
    const int64_t t = index[r];
    return t < 0 ? 0 : (t >= x_rows ? x_rows - 1 : t);
}

// One unit of grouped-GEMM work: `rows` rows starting at `row0`, all of expert `e`.
struct MTile {
    int e;
    int rows;        // 0 => no work for this block
    int64_t row0;
};

// Finds the `tile`-th row tile of height BM in expert order, straight from expert_offset.
// Every wave works it out for itself, four experts per lane (E <= 256): tile counts per expert,
// a prefix sum over the lanes, one ballot for the lane that owns the tile -- no LDS, no block
// barrier, and no walk over the experts by every thread (with 256 experts that walk took longer
// than a short block's whole K loop).  Offsets are clamped into [0, R] and a segment that ends
// before it starts counts as empty, so a corrupt offset can never send a store outside Y.
// Every thread of the block must call it (whole waves, converged).
__device__ __forceinline__ MTile find_mtile(const int64_t *__restrict__ off, int E, int64_t R, int BM, int64_t tile)
{
    static_assert(OPMX_MOE_MAX_EXPERTS <= 4 * kWave, "four experts per lane");
    MTile t;
    t.e = 0;
    t.rows = 0;
    t.row0 = 0;
    if (off == nullptr) {               // dense GEMM: one "expert" owns rows [0, R)
        t.row0 = tile * BM;
        const int64_t left = R - t.row0;
        t.rows = left <= 0 ? 0 : static_cast<int>(left < BM ? left : BM);
        return t;
    }
    const int lane = threadIdx.x & (kWave - 1);
    int64_t o[5];
#pragma unroll
    for (int j = 0; j < 5; ++j) {
        const int idx = lane * 4 + j;
        const int64_t v = off[idx < E ? idx : E];
        o[j] = v < 0 ? 0 : (v > R ? R : v);
    }
    int nt[4], tot = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t rows = o[j + 1] - o[j];
        nt[j] = (lane * 4 + j < E && rows > 0) ? static_cast<int>((rows + BM - 1) / BM) : 0;
        tot += nt[j];
    }
    int incl = tot;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += up;
    }
    const int excl = incl - tot;
    const int want = tile < (int64_t{1} << 31) ? static_cast<int>(tile) : 0x7fffffff;
    const uint64_t owner = __ballot(want >= excl && want < incl);
    if (owner == 0) return t;           // past the last tile (uniform)
    const int src = __ffsll(static_cast<long long>(owner)) - 1;
    // the owning lane picks the expert among its four
    int e_local = 3, before = excl + nt[0] + nt[1] + nt[2];
    if (want < excl + nt[0]) {
        e_local = 0;
        before = excl;
    } else if (want < excl + nt[0] + nt[1]) {
        e_local = 1;
        before = excl + nt[0];
    } else if (want < excl + nt[0] + nt[1] + nt[2]) {
        e_local = 2;
        before = excl + nt[0] + nt[1];
    }
    const int64_t lo = e_local == 0 ? o[0] : e_local == 1 ? o[1] : e_local == 2 ? o[2] : o[3];
    const int64_t hi = e_local == 0 ? o[1] : e_local == 1 ? o[2] : e_local == 2 ? o[3] : o[4];
    const int64_t row0 = lo + static_cast<int64_t>(want - before) * BM, left = hi - row0;
    const int rows = static_cast<int>(left < BM ? left : BM);
    // block-uniform by construction; say so to the compiler (scalar registers)
    t.e = __builtin_amdgcn_readlane(lane * 4 + e_local, src);
    t.row0 = (static_cast<int64_t>(__builtin_amdgcn_readlane(static_cast<int>(row0 >> 32), src)) << 32) |
             static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(row0), src));
    t.rows = __builtin_amdgcn_readlane(rows, src);
    return t;
}

// Upper bound of the number of row tiles for any offsets: sum ceil(m_e/BM) <= R/BM + E, and
// never more than R, as every tile holds at least one row (a single token routed to 8 of 64
// experts: 8 tiles, not 64 -- the blocks of the others would start only to find no work).
inline int64_t max_mtiles(int64_t R, int E, int BM)
{
    const int64_t bound = R / BM + E;
    return bound < R ? bound : R;
}

// Rows outside [off[0], off[E]) belong to no expert and must read as zero
// (MoeColumnParallelLinear.py:59 starts from torch.zeros).  Normally there are
// none and this is two loads.  Work is shared by all blocks of the grid.
template <typename T>
__device__ __forceinline__ void zero_unowned_rows(T *__restrict__ Y, int64_t R, int64_t ncols,
                                                  const int64_t *__restrict__ off, int E)
{
    if (off == nullptr) return;
    int64_t lo = off[0], hi = off[E];
    lo = lo < 0 ? 0 : (lo > R ? R : lo);
    hi = hi < lo ? lo : (hi > R ? R : hi);
    const int64_t head = lo * ncols, tail0 = hi * ncols, total = R * ncols;
    if (head == 0 && tail0 == total) return;
    const int64_t nb = static_cast<int64_t>(gridDim.x) * gridDim.y * gridDim.z;
    const int64_t b = blockIdx.x + static_cast<int64_t>(gridDim.x) * (blockIdx.y + static_cast<int64_t>(gridDim.y) * blockIdx.z);
    const int64_t stride = nb * blockDim.x;
    for (int64_t i = b * blockDim.x + threadIdx.x; i < head; i += stride) Y[i] = from_f32<T>(0.0f);
    for (int64_t i = tail0 + b * blockDim.x + threadIdx.x; i < total; i += stride) Y[i] = from_f32<T>(0.0f);
}

int launch_gemm_generic(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                        int64_t K, int64_t N, int dtype, int epilogue, void *Y, hipStream_t s, RowGather g = {});
// fp32 tensors on the fp32 matrix units; requires K % 4 == 0 and 16-byte aligned X and W.
int launch_gemm_f32(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R, int64_t K,
                    int64_t N, int epilogue, int64_t rows_hint, void *Y, hipStream_t s, RowGather g = {});
// variant: 0 = 256x256 direct-to-LDS kernel, 1 = 256x256 register-staged (8 waves),
// 2 = 128x128 register-staged (4 waves).  off == nullptr: dense GEMM (one expert owns [0, R)).
// ws / ws_bytes: optional scratch memory of gemm_tiled_workspace_bytes() bytes (variant 0 then
// balances the last rounds of tiles over all CUs); nullptr / 0 is always accepted.
int launch_gemm_tiled(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                      int64_t K, int64_t N, int dtype, int epilogue, int variant, void *Y, void *ws,
                      size_t ws_bytes, hipStream_t s, RowGather g = {});
size_t gemm_tiled_workspace_bytes();
int launch_grouped_gemm(const void *X, const int64_t *off, const void *W, const void *B, int E,
                        int64_t R, int64_t K, int64_t N, int dtype, int epilogue, int64_t rows_hint,
                        void *Y, void *ws, size_t ws_bytes, hipStream_t s, RowGather g = {});
int launch_gemm_stream(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                       int64_t K, int64_t N, int dtype, int epilogue, int64_t rows_hint, int variant, void *Y,
                       hipStream_t s, RowGather g = {});

}  // namespace opmx
