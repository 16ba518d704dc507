// Device-ceiling probe for MI355X: what this GPU sustains for (a) a pure streaming
// read of a weight-sized buffer and (b, c) MFMA loops (32x32x16 and 16x16x32) on random fp16
// operands, register-fed and LDS-fed, and (d) what one CU pulls into LDS in the tile kernels'
// operand shape (two 256-row x 128-byte k-tiles per step, rows 2*K bytes apart, fetched with
// buffer_load ... lds and nothing else going on): once with every workgroup re-reading tiles
// that stay in L2, once as 32 workgroups per XCD walk K as an 8 x 4 block of output tiles
// does (each X tile shared by 4, each W tile by 8, all of it new to the L2 at every step).
// These are the practical ceilings the grouped-GEMM
// kernels are compared with in addition to the vendor peaks (8 TB/s, 2.5 PFLOP/s):
// the engine clock drops under dense MFMA load with toggling operands, so the vendor
// MFMA peak is not reachable by any kernel on real data.
// Prints one JSON object.  Build: see Makefile (target ../lib/opmx_device_ceilings).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                              \
    do {                                                                      \
        hipError_t e_ = (x);                                                  \
        if (e_ != hipSuccess) {                                               \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));           \
            return 1;                                                         \
        }                                                                     \
    } while (0)

// ---- (a) streaming read: every block reads one contiguous slab, 16 KiB in flight per wave
template <bool NT>
__global__ __launch_bounds__(256) void read_kernel(const u32x4 *__restrict__ src, size_t n16_per_block, unsigned *out)
{
    const u32x4 *p = src + static_cast<size_t>(blockIdx.x) * n16_per_block;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = threadIdx.x; i + 15 * 256 < n16_per_block; i += 256 * 16) {
        u32x4 v[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) v[u] = NT ? __builtin_nontemporal_load(p + i + u * 256) : p[i + u * 256];
#pragma unroll
        for (int u = 0; u < 16; ++u) acc ^= v[u];
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) out[0] = 1;
}

// ---- (b) MFMA 32x32x16 f16 on random operands; LDS_FED: 6 ds_read_b128 per 8 MFMAs
// (the fragment traffic of a 128x64 wave tile), else two fixed register fragments
template <bool LDS_FED>
__global__ __launch_bounds__(512) void mfma_kernel(const _Float16 *__restrict__ src, float *out, int iters)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x;
    for (int i = tid; i < 65536 / 16; i += blockDim.x)
        reinterpret_cast<u32x4 *>(smem)[i] = reinterpret_cast<const u32x4 *>(src)[i + (blockIdx.x & 7) * 4096];
    __syncthreads();
    const half8 ra = *reinterpret_cast<const half8 *>(smem + (tid * 16) % 65536);
    const half8 rb = *reinterpret_cast<const half8 *>(smem + (tid * 16 + 32768) % 65536);
    float16v acc[8];
    for (int j = 0; j < 8; ++j)
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;
    const int base = (tid >> 6) * 4096 + (tid & 63) * 16;
    for (int it = 0; it < iters; ++it) {
        if (LDS_FED) {
            half8 fa[4], fb[2];
            const int o = (base + (it & 15) * 3072) & 65520;
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = *reinterpret_cast<const half8 *>(smem + ((o + i * 1024) & 65535));
#pragma unroll
            for (int i = 0; i < 2; ++i) fb[i] = *reinterpret_cast<const half8 *>(smem + ((o + 32768 + i * 1024) & 65535));
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i * 2 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i * 2 + j], 0, 0, 0);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ra, rb, acc[j], 0, 0, 0);
        }
    }
    float s = 0;
    for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][7];
    out[blockIdx.x * blockDim.x + tid] = s;
}

// ---- (c) the same for MFMA 16x16x32 f16 (the grouped-GEMM kernels' instruction); LDS_FED:
// 12 ds_read_b128 per 32 MFMAs, the same fragment bytes per flop as above
typedef float float4v __attribute__((ext_vector_type(4)));
template <bool LDS_FED>
__global__ __launch_bounds__(512) void mfma16_kernel(const _Float16 *__restrict__ src, float *out, int iters)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x;
    for (int i = tid; i < 65536 / 16; i += blockDim.x)
        reinterpret_cast<u32x4 *>(smem)[i] = reinterpret_cast<const u32x4 *>(src)[i + (blockIdx.x & 7) * 4096];
    __syncthreads();
    float4v acc[32];
    for (int j = 0; j < 32; ++j)
        for (int v = 0; v < 4; ++v) acc[j][v] = 0.f;
    const int base = (tid >> 6) * 4096 + (tid & 63) * 16;
    half8 fa[2][8], fb[2][4];
    auto rd = [&](int set, int it) {
        const int o = (base + (it & 15) * 3072) & 65520;
#pragma unroll
        for (int i = 0; i < 8; ++i) fa[set][i] = *reinterpret_cast<const half8 *>(smem + ((o + i * 1024) & 65535));
#pragma unroll
        for (int i = 0; i < 4; ++i) fb[set][i] = *reinterpret_cast<const half8 *>(smem + ((o + 32768 + i * 1024) & 65535));
    };
    rd(0, 0);
    rd(1, 1);
    for (int it = 0; it < iters; it += 2) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (LDS_FED) rd((h + 1) & 1, it + h + 1);
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[h][i], fb[h][j], acc[i * 4 + j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0;
    for (int j = 0; j < 32; ++j) s += acc[j][0] + acc[j][3];
    out[blockIdx.x * blockDim.x + tid] = s;
}

// ---- (d) operand pull of a 256x256 output tile: per step eight 1 KiB wave loads per wave
// (four of the X tile, four of the W tile) straight into LDS, the next step issued while one
// is in flight.  resident: every workgroup re-reads one k-tile of its own.
#define LPTR(p) ((void __attribute__((address_space(3))) *)(p))
__global__ __launch_bounds__(512) void pull_kernel(const char *xbase, const char *wbase, uint32_t ld, int ktiles,
                                                   int steps, bool resident, unsigned *out)
{
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;   // workgroups go round the XCDs
    const size_t tile = 256 * static_cast<size_t>(ld);
    const char *xp = xbase + (resident ? blockIdx.x & 63 : xcd * 8 + (slot >> 2)) * tile;
    const char *wp = wbase + (resident ? blockIdx.x & 63 : xcd * 4 + (slot & 3)) * tile;
    auto descriptor = [](const char *base) {
        const uint64_t b = reinterpret_cast<uint64_t>(base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32));
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>((static_cast<uint64_t>(hi) << 32) | lo),
                                                 0, static_cast<int>(0xFFFFFFFFu), 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t xr = descriptor(xp), wr = descriptor(wp);
    uint32_t voff[4];
    for (int i = 0; i < 4; ++i) voff[i] = (8 * (wave * 4 + i) + (lane >> 3)) * ld + (lane & 7) * 16;
    int kt = 0;
    for (int s = 0; s < steps; ++s) {
        const int soff = resident ? (blockIdx.x >> 6) * 128 : kt * 128;
        char *buf = smem + (s & 1) * 65536 + wave * 8192;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, LPTR(buf + i * 1024), 16, voff[i], soff, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, LPTR(buf + 4096 + i * 1024), 16, voff[i], soff, 0, 0);
        }
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        if (++kt == ktiles) kt = 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (reinterpret_cast<unsigned *>(smem)[tid] == 0x12345678u) out[0] = 1;
}

static float best_ms(hipEvent_t e0, hipEvent_t e1, int reps, void (*launch)(void *), void *ctx)
{
    float best = 1e30f;
    for (int r = 0; r < reps; ++r) {
        (void)hipEventRecord(e0);
        launch(ctx);
        (void)hipEventRecord(e1);
        (void)hipEventSynchronize(e1);
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        if (r > 0 && ms < best) best = ms;   // first repetition is warm-up
    }
    return best;
}

struct ReadCtx { const u32x4 *src; size_t n16; unsigned *out; int blocks; bool nt; };
struct PullCtx { const char *x, *w; uint32_t ld; int ktiles, steps; bool resident; unsigned *out; };
struct MfmaCtx { const _Float16 *src; float *out; int iters; bool lds; bool m16; };

int main()
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    // (a)
    const size_t bytes = 1879048192ull;   // one Mixtral-8x7B gate/up weight tensor
    u32x4 *buf;
    unsigned *flag;
    CHECK(hipMalloc(&buf, bytes));
    CHECK(hipMemset(buf, 1, bytes));
    CHECK(hipMalloc(&flag, 4));
    const int blocks = 2048;
    ReadCtx rc{buf, bytes / 16 / blocks, flag, blocks, false};
    auto read_launch = [](void *c) {
        ReadCtx *r = static_cast<ReadCtx *>(c);
        if (r->nt) read_kernel<true><<<r->blocks, 256>>>(r->src, r->n16, r->out);
        else read_kernel<false><<<r->blocks, 256>>>(r->src, r->n16, r->out);
    };
    const double read_plain = bytes / best_ms(e0, e1, 4, read_launch, &rc) / 1e6;
    rc.nt = true;
    const double read_nt = bytes / best_ms(e0, e1, 4, read_launch, &rc) / 1e6;
    // (b)
    const size_t n = 1 << 20;
    std::vector<_Float16> h(n);
    srand(1);
    for (size_t i = 0; i < n; ++i) h[i] = static_cast<_Float16>(((rand() % 2001) - 1000) * 0.002f);
    _Float16 *src;
    float *out;
    CHECK(hipMalloc(&src, n * 2));
    CHECK(hipMemcpy(src, h.data(), n * 2, hipMemcpyHostToDevice));
    CHECK(hipMalloc(&out, 256 * 512 * 4));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mfma_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mfma_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mfma16_kernel<true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mfma16_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    MfmaCtx mc{src, out, 8000, false, false};
    auto mfma_launch = [](void *c) {
        MfmaCtx *m = static_cast<MfmaCtx *>(c);
        if (m->m16) {
            if (m->lds) mfma16_kernel<true><<<256, 512, 65536>>>(m->src, m->out, m->iters);
            else mfma16_kernel<false><<<256, 512, 65536>>>(m->src, m->out, m->iters);
        } else {
            if (m->lds) mfma_kernel<true><<<256, 512, 65536>>>(m->src, m->out, m->iters);
            else mfma_kernel<false><<<256, 512, 65536>>>(m->src, m->out, m->iters);
        }
    };
    const double flops = 256.0 * 8 * mc.iters * 8 * 32768.0;
    const double mfma_reg = flops / best_ms(e0, e1, 5, mfma_launch, &mc) / 1e9;
    mc.lds = true;
    const double mfma_lds = flops / best_ms(e0, e1, 5, mfma_launch, &mc) / 1e9;
    // 16x16x32: 32 MFMAs of 16384 flops per iteration, same flops per iteration count as above
    mc.m16 = true;
    mc.lds = false;
    mc.iters = 4000;
    const double flops16 = 256.0 * 8 * mc.iters * 32 * 16384.0;
    const double mfma16_reg = flops16 / best_ms(e0, e1, 5, mfma_launch, &mc) / 1e9;
    mc.lds = true;
    const double mfma16_lds = flops16 / best_ms(e0, e1, 5, mfma_launch, &mc) / 1e9;
    // (d): 64 X tiles and 32 W tiles of 256 rows x K = 14336 fp16 (the down projection's K)
    const uint32_t pull_ld = 14336 * 2;
    const size_t pull_tile = 256 * static_cast<size_t>(pull_ld);
    char *px, *pw;
    CHECK(hipMalloc(&px, 64 * pull_tile));
    CHECK(hipMalloc(&pw, 64 * pull_tile));
    CHECK(hipMemset(px, 1, 64 * pull_tile));
    CHECK(hipMemset(pw, 2, 64 * pull_tile));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(pull_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              131072));
    PullCtx pc{px, pw, pull_ld, static_cast<int>(pull_ld / 128), 4000, true, flag};
    auto pull_launch = [](void *c) {
        PullCtx *p = static_cast<PullCtx *>(c);
        pull_kernel<<<256, 512, 131072>>>(p->x, p->w, p->ld, p->ktiles, p->steps, p->resident, p->out);
    };
    const double pull_resident = 65536.0 * pc.steps / best_ms(e0, e1, 4, pull_launch, &pc) / 1e6;
    pc.resident = false;
    const double pull_streamed = 65536.0 * pc.steps / best_ms(e0, e1, 4, pull_launch, &pc) / 1e6;
    CHECK(hipGetLastError());
    printf("{\"hbm_read_GBs\": %.0f, \"hbm_read_nontemporal_GBs\": %.0f, "
           "\"mfma_f16_register_fed_TFLOPs\": %.0f, \"mfma_f16_lds_fed_TFLOPs\": %.0f, "
           "\"mfma_f16_16x16x32_register_fed_TFLOPs\": %.0f, \"mfma_f16_16x16x32_lds_fed_TFLOPs\": %.0f, "
           "\"tile_operands_to_lds_L2_resident_GBs_per_CU\": %.1f, "
           "\"tile_operands_to_lds_streamed_8x4_per_XCD_GBs_per_CU\": %.1f}\n",
           read_plain, read_nt, mfma_reg, mfma_lds, mfma16_reg, mfma16_lds, pull_resident, pull_streamed);
    return 0;
}
