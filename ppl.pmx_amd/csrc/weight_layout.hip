// Expert weights in the layout the weight-streaming kernels read fastest.
//
// Reference layout: W[e] is [N, K] row-major (model_zoo/ModelParallel.py:149-151 of
// OpenPPL/ppl.pmx; checkpoints from model_zoo/mixtral/huggingface/ConvertWeightToOpmx.py:98-128).
// A wave of the streaming kernel owns 16 rows of W[e] and walks K: in that layout every 1 KiB
// wave load is two to four pieces of 256-512 bytes, K*2 bytes apart, and the memory system
// serves the stream 7-9 % below what it gives for one contiguous run.
//
// Tiled layout ("16 x 64 tiles"): W[e] cut into tiles of 16 rows x 64 k (2 KiB each), stored
// tile after tile, k fastest: element (n, k) of expert e lives at element offset
//     e*N*K + ((n/16) * (K/64) + k/64) * 1024 + (n%16) * 64 + k%64.
// The 16 rows of a wave are then one contiguous run of 32*K bytes.  Needs N % 16 == 0 and
// K % 64 == 0, 2-byte elements.  The conversion is a permutation of 16-byte chunks, done once
// when the weights are loaded; every grouped-GEMM kernel of the library reads either layout.
#include "common.h"

namespace opmx {
namespace {

template <bool TO_TILED>
__global__ __launch_bounds__(256) void retile_kernel(const uint4 *__restrict__ in, uint4 *__restrict__ out,
                                                     int64_t chunks, int64_t per_expert, int64_t ktiles, int64_t krow)
{
    // q: index of a 16-byte chunk of the TILED tensor; per_expert = N*K/8, krow = K/8 chunks per row
    for (int64_t q = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; q < chunks;
         q += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t e = q / per_expert, rem = q - e * per_expert;
        const int64_t tile = rem >> 7, c = rem & 127;            // 128 chunks per 2 KiB tile
        const int64_t nb = tile / ktiles, kt = tile - nb * ktiles;
        const int64_t row = nb * 16 + (c >> 3);
        const int64_t rm = e * per_expert + row * krow + kt * 8 + (c & 7);
        if (TO_TILED) out[q] = in[rm];
        else out[rm] = in[q];
    }
}

}  // namespace

int launch_retile_weights(const void *in, int E, int64_t N, int64_t K, int dtype, int to_tiled, void *out,
                          hipStream_t s)
{
    if (dtype != OPMX_DTYPE_F16 && dtype != OPMX_DTYPE_BF16) return OPMX_ERR_UNSUPPORTED;
    if (N % 16 != 0 || K % 64 != 0) return OPMX_ERR_UNSUPPORTED;
    if (!aligned16(in) || !aligned16(out)) return OPMX_ERR_ALIGNMENT;
    const int64_t per_expert = N * K / 8, chunks = per_expert * E;
    if (chunks == 0) return OPMX_OK;
    int64_t blocks = ceil_div(chunks, 256);
    if (blocks > 65536) blocks = 65536;
    const uint4 *src = static_cast<const uint4 *>(in);
    uint4 *dst = static_cast<uint4 *>(out);
    if (to_tiled)
        retile_kernel<true><<<static_cast<unsigned>(blocks), 256, 0, s>>>(src, dst, chunks, per_expert, K / 64, K / 8);
    else
        retile_kernel<false><<<static_cast<unsigned>(blocks), 256, 0, s>>>(src, dst, chunks, per_expert, K / 64, K / 8);
    OPMX_LAUNCH_CHECK();
    return OPMX_OK;
}

}  // namespace opmx
