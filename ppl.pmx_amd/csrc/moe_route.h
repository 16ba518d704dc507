// Top-k routing of one token by a group of lanes, shared by the MoeSelect kernels and by the
// router-gate kernel that routes in its epilogue.  Semantics: torch_function/MoeSelect.py:40-41 of
// OpenPPL/ppl.pmx with ties going to the lower expert id.
#pragma once
#include "common.h"

namespace opmx {
namespace {

constexpr int kMaxVpl = OPMX_MOE_MAX_EXPERTS / kWave;

// Monotone map float -> uint32 (larger float => larger key).  NaN is the
// largest key (torch.topk / torch.sort rank NaN first); -0.0 == +0.0.
__device__ __forceinline__ uint32_t order_key(float f)
{
    if (f != f) return 0xFFFFFFFFu;
    if (f == 0.0f) f = 0.0f;
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key)
{
    if (key == 0xFFFFFFFFu) return __uint_as_float(0x7FC00000u);
    uint32_t u = (key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key;
    return __uint_as_float(u);
}

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask)
{
    uint32_t lo = __shfl_xor(static_cast<uint32_t>(v), mask, kWave);
    uint32_t hi = __shfl_xor(static_cast<uint32_t>(v >> 32), mask, kWave);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// One group of G lanes (G a power of two, 8..64) routes one token.  Lane j < k
// of the group ends up with the j-th pick and its softmax weight.
template <typename T>
__device__ __forceinline__ void route_token(const T *srow, int E, int k, int G, int vpl, int lig,
                                            int &my_id, float &my_w)
{
    uint64_t keys[kMaxVpl];
#pragma unroll
    for (int v = 0; v < kMaxVpl; ++v) {
        int e = lig + v * G;
        keys[v] = (v < vpl && e < E)
                      ? (static_cast<uint64_t>(order_key(to_f32(srow[e]))) << 32) | (0xFFFFFFFFu - e)
                      : 0ull;
    }
    my_id = -1;
    float my_v = 0.0f;
    // With several keys per lane (E > 64) the ranking below costs E broadcasts of up to four
    // compares each; the k rounds of the other branch are cheaper there (E = 256, k = 8: MoeSelect at
    // T = 512 51 -> 38 us, at T = 8192 291 -> 247 us), so only one key per lane is ranked.
    if (G == kWave && vpl == 1) {
        // A whole wave routes the token.  Keys are distinct (the id is part of the key),
        // so "how many keys beat mine" is the key's position in the descending order:
        // E scalar broadcasts and compares, no k-round dependency chain.  The key of
        // rank j then moves to lane j through LDS-free cross-lane reads.
        int rank = 0;
        for (int sl = 0; sl < E; ++sl) {
            const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(keys[0]), sl);
            const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(keys[0] >> 32), sl);
            rank += ((static_cast<uint64_t>(hi) << 32) | lo) > keys[0] ? 1 : 0;
        }
        // lane j < k fetches the key whose rank is j: every lane publishes (rank -> key) by ballot
        for (int j = 0; j < k; ++j) {
            const uint64_t hit = __ballot(rank == j && keys[0] != 0ull);
            if (hit) {
                const int src = __ffsll(static_cast<long long>(hit)) - 1;
                const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(keys[0]), src);
                const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(keys[0] >> 32), src);
                if (lig == j) {
                    my_id = static_cast<int>(0xFFFFFFFFu - lo);
                    my_v = key_value(hi);
                }
            }
        }
    } else {
        for (int j = 0; j < k; ++j) {
            uint64_t best = keys[0];
#pragma unroll
            for (int v = 1; v < kMaxVpl; ++v) best = keys[v] > best ? keys[v] : best;
            for (int m = G >> 1; m >= 1; m >>= 1) {
                uint64_t o = shfl_xor_u64(best, m);
                best = o > best ? o : best;
            }
            int wid = static_cast<int>(0xFFFFFFFFu - static_cast<uint32_t>(best));
#pragma unroll
            for (int v = 0; v < kMaxVpl; ++v)
                if (lig + v * G == wid) keys[v] = 0ull;
            if (lig == j) {
                my_id = wid;
                my_v = key_value(static_cast<uint32_t>(best >> 32));
            }
        }
    }
    // softmax over the k picked values (MoeSelect.py:41); pick 0 is the maximum
    float vmax = __shfl(my_v, (lane_id() / G) * G, kWave);
    float ev = (lig < k) ? expf(my_v - vmax) : 0.0f;
    float sum = ev;
    for (int m = G >> 1; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, kWave);
    my_w = ev / sum;
}

}  // namespace
}  // namespace opmx
