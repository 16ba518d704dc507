// extern "C" surface of libopmx_moe.so: argument checks and kernel selection.
// Declarations and the reference operator each entry point replaces are in
// include/opmx_moe.h.
#include <atomic>
#include <cstdlib>
#include <cstring>

#include "moe_gemm.h"

using namespace opmx;

namespace {

inline bool dtype_ok(int d) { return d == OPMX_DTYPE_F32 || d == OPMX_DTYPE_F16 || d == OPMX_DTYPE_BF16; }
inline size_t elt(int d) { return d == OPMX_DTYPE_F32 ? 4 : 2; }
inline hipStream_t st(void *s) { return static_cast<hipStream_t>(s); }

// The weight-streaming kernel wins while a row tile of twice the mean rows per expert is
// at most 64 rows (measured crossover against the 128x256 MFMA tiles on MI355X).
constexpr int64_t kStreamMaxRowsPerExpert = 64;

const char *const kOptionNames[kNumOptions] = {"OPMX_MOE_GEMM", "OPMX_MOE_GEMM_TILED_VARIANT",
                                               "OPMX_MOE_GEMM_STREAM_VARIANT", "OPMX_MOE_GEMM_GNX",
                                               "OPMX_MOE_GEMM_STREAMK", "OPMX_MOE_GEMM_PERSIST",
                                               "OPMX_MOE_ROUTE_INDEX_TOKENS", "OPMX_MOE_GEMM_F32_VARIANT"};

// Kernel family names accepted for OPMX_MOE_GEMM in the environment.
int parse_option(int id, const char *v)
{
    if (!v || !*v) return -1;
    if (id == kOptGemm) {
        if (!std::strcmp(v, "generic")) return 1;
        if (!std::strcmp(v, "tiled")) return 2;
        if (!std::strcmp(v, "stream")) return 3;
    }
    char *end = nullptr;
    const long n = std::strtol(v, &end, 10);
    return (end && *end == 0 && n >= 0 && n < 1000) ? static_cast<int>(n) : -1;
}

// The knobs: filled from the environment when first needed (thread-safe: initialisation of a
// function-local static), changed afterwards only through opmx_moe_set_option.
struct Options {
    std::atomic<int> v[kNumOptions];
    Options()
    {
        for (int i = 0; i < kNumOptions; ++i) v[i].store(parse_option(i, std::getenv(kOptionNames[i])));
    }
};
Options &options()
{
    static Options o;
    return o;
}

std::atomic<int> g_cu_count[kMaxDevices];

}  // namespace

namespace opmx {

int option(Option o) { return options().v[o].load(std::memory_order_relaxed); }

int cu_count()
{
    const int dev = current_device();
    if (dev < 0) return 0;
    int n = g_cu_count[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        g_cu_count[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Scratch memory that lets the 256x256 tile kernel balance its last rounds of tiles over all
// CUs (stream-K); every kernel also runs without it.  256 bytes when the call would not use it.
size_t grouped_gemm_workspace_bytes(int E, int64_t R, int64_t K, int64_t N, int dtype)
{
    (void)N;
    const bool lowp = dtype == OPMX_DTYPE_F16 || dtype == OPMX_DTYPE_BF16;
    if (lowp && E > 0 && K > 0 && K % 64 == 0 && 2 * ceil_div(R, E) > kStreamMaxRowsPerExpert) {
        const size_t b = gemm_tiled_workspace_bytes();
        if (b > 0) return (b + 255) / 256 * 256;
    }
    return 256;
}

int launch_grouped_gemm(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                        int64_t K, int64_t N, int dtype, int epilogue, int64_t rows_hint, void *Y, void *ws,
                        size_t ws_bytes, hipStream_t s, RowGather g)
{
    const int64_t ncols = epilogue == OPMX_EPILOGUE_SWIGLU ? N / 2 : N;
    if (R == 0 || ncols == 0) return OPMX_OK;
    const bool lowp = dtype == OPMX_DTYPE_F16 || dtype == OPMX_DTYPE_BF16;
    // (through a row index the MFMA kernels address X with 32-bit byte offsets)
    const bool mfma_ok = lowp && K > 0 && K % 8 == 0 && aligned16(X) && aligned16(W) &&
                         N * K < (int64_t{1} << 31) && R * K < (int64_t{1} << 40) &&
                         (g.index == nullptr || g.x_rows * K * 2 < (int64_t{1} << 31));
    const bool tiled_ok = mfma_ok && K % 64 == 0;
    // Row-tile sizing: twice the mean rows per expert, never above what the caller can
    // guarantee.  An expert with more rows than one tile simply takes several tiles.
    int64_t hint = rows_hint > 0 && rows_hint < R ? rows_hint : R;
    const int64_t twice_mean = 2 * ceil_div(R, E);
    if (twice_mean < hint) hint = twice_mean;
    const bool stream_ws = true;   // the stream kernel needs no scratch memory
    const int force = option(kOptGemm);      // 1 generic, 2 tiled, 3 stream, else automatic

    int choice;   // 1 generic, 2 tiled, 3 stream
    if (force == 3 && mfma_ok && stream_ws) choice = 3;
    else if (force == 2 && tiled_ok) choice = 2;
    else if (force == 1) choice = 1;
    else if (mfma_ok && stream_ws && hint <= kStreamMaxRowsPerExpert) choice = 3;
    else if (tiled_ok) choice = 2;
    else if (mfma_ok && stream_ws) choice = 3;   // K a multiple of 8 but not of 64: 128-row tiles of the stream kernel
    else choice = 1;                             // (MFMA, weights re-read per row tile) rather than the FMA fallback

    if (choice == 3)
        return launch_gemm_stream(X, off, W, B, E, R, K, N, dtype, epilogue, hint,
                                  option(kOptStreamVariant) < 0 ? 0 : option(kOptStreamVariant), Y, s, g);
    if (choice == 2) {
        // The direct-to-LDS kernel takes 256x256 tiles unless they would fill the CUs less than
        // twice (the Mixtral down projection at T=2048: 1.3 rounds) or the experts hold fewer than
        // 128 rows on average: then 128x256 tiles, 20 % slower per flop but with half the
        // quantisation (-9 % at T=2048; at T=256 8 % faster than 128x128 register-staged tiles).
        const int64_t out_cols = epilogue == OPMX_EPILOGUE_SWIGLU ? N / 2 : N;
        const int64_t tiles256 = (R / 256 + (E + 1) / 2) * ((out_cols + 255) / 256);
        const int dflt = R / E >= 128 && tiles256 >= 512 ? 0 : 3;
        return launch_gemm_tiled(X, off, W, B, E, R, K, N, dtype, epilogue,
                                 option(kOptTiledVariant) < 0 ? dflt : option(kOptTiledVariant), Y, ws, ws_bytes, s, g);
    }
    // fp32 tensors: the fp32 matrix-unit kernel where its alignment conditions hold
    if (dtype == OPMX_DTYPE_F32 && force != 1 && K > 0 && K % 4 == 0 && aligned16(X) && aligned16(W))
        return launch_gemm_f32(X, off, W, B, E, R, K, N, epilogue, hint, Y, s, g);
    return launch_gemm_generic(X, off, W, B, E, R, K, N, dtype, epilogue, Y, s, g);
}

}  // namespace opmx

extern "C" {

int opmx_moe_abi_version(void) { return OPMX_MOE_ABI_VERSION; }

int opmx_moe_set_option(const char *name, int value)
{
    if (!name) return OPMX_ERR_BAD_ARGUMENT;
    for (int i = 0; i < kNumOptions; ++i)
        if (!std::strcmp(name, kOptionNames[i])) {
            options().v[i].store(value < 0 ? -1 : value, std::memory_order_relaxed);
            return OPMX_OK;
        }
    return OPMX_ERR_BAD_ARGUMENT;
}

const char *opmx_status_string(int status)
{
    switch (status) {
        case OPMX_OK: return "ok";
        case OPMX_ERR_BAD_ARGUMENT: return "bad argument";
        case OPMX_ERR_UNSUPPORTED: return "unsupported dtype, expert count or experts-per-token";
        case OPMX_ERR_WORKSPACE: return "workspace missing or too small";
        case OPMX_ERR_ALIGNMENT: return "pointer or row pitch not aligned";
        case OPMX_ERR_LAUNCH: return "HIP launch failed";
    }
    return "unknown status";
}

int opmx_linear(const void *X, const void *W, const void *B, int64_t T, int64_t K, int64_t N, int dtype,
                void *Y, void *stream)
{
    if (T < 0 || K < 0 || N < 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype)) return OPMX_ERR_UNSUPPORTED;
    if (T == 0 || N == 0) return OPMX_OK;
    if (!X || !W || !Y || K == 0) return OPMX_ERR_BAD_ARGUMENT;
    return launch_linear(X, W, B, T, K, N, dtype, Y, st(stream));
}

size_t opmx_moe_select_workspace_bytes(int64_t T, int E, int k) { return moe_select_workspace_bytes(T, E, k); }

int opmx_moe_select(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                    void *X_expand_permute, void *expert_weights, int64_t *invert_permutation,
                    int64_t *expert_offset, int32_t *expert_ids, void *workspace, size_t workspace_bytes,
                    void *stream)
{
    if (T < 0 || H < 0 || E <= 0 || k <= 0 || k > E) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN)
        return OPMX_ERR_UNSUPPORTED;
    if (T > (int64_t{1} << 31) / k) return OPMX_ERR_UNSUPPORTED;
    if (!expert_offset) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!scores || !expert_weights || !invert_permutation)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && H > 0 && (!X || !X_expand_permute)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!workspace || workspace_bytes < moe_select_workspace_bytes(T, E, k))) return OPMX_ERR_WORKSPACE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OPMX_ERR_ALIGNMENT;
    return launch_moe_select(X, scores, T, H, E, k, dtype, X_expand_permute, expert_weights, invert_permutation,
                             expert_offset, expert_ids, workspace, st(stream));
}

int opmx_moe_select_static(const void *X, const void *scores, int64_t T, int64_t H, int E, int k, int dtype,
                           void *X_expand_permute, void *expert_weights, int64_t *invert_permutation,
                           int64_t *expert_offset, int32_t *expert_ids, void *stream)
{
    if (T < 0 || H < 0 || E <= 0 || k <= 0 || k > E) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN)
        return OPMX_ERR_UNSUPPORTED;
    if (T > (int64_t{1} << 31) / k) return OPMX_ERR_UNSUPPORTED;
    if (!expert_offset) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!scores || !expert_weights || !invert_permutation)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && H > 0 && (!X || !X_expand_permute)) return OPMX_ERR_BAD_ARGUMENT;
    // more tokens than the library's own scratch memory holds: rejected on the host
    if (moe_select_workspace_bytes(T, E, k) > OPMX_MOE_SELECT_STATIC_SCRATCH_BYTES) return OPMX_ERR_WORKSPACE;
    return launch_moe_select_static(X, scores, T, H, E, k, dtype, X_expand_permute, expert_weights,
                                    invert_permutation, expert_offset, expert_ids, st(stream));
}

int opmx_moe_route_select(const void *X, const void *gate_weight, const void *gate_bias, int64_t T, int64_t H, int E,
                          int k, int dtype, void *scores, void *X_expand_permute, void *expert_weights,
                          int64_t *invert_permutation, int64_t *expert_offset, int32_t *expert_ids, void *workspace,
                          size_t workspace_bytes, void *stream)
{
    if (T < 0 || H < 0 || E <= 0 || k <= 0 || k > E) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN)
        return OPMX_ERR_UNSUPPORTED;
    if (T > (int64_t{1} << 31) / k) return OPMX_ERR_UNSUPPORTED;
    if (!expert_offset) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!scores || !expert_weights || !invert_permutation)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && H > 0 && (!X || !gate_weight || !X_expand_permute)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!workspace || workspace_bytes < moe_select_workspace_bytes(T, E, k))) return OPMX_ERR_WORKSPACE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OPMX_ERR_ALIGNMENT;
    return launch_moe_route_select(X, gate_weight, gate_bias, T, H, E, k, dtype, scores, X_expand_permute,
                                   expert_weights, invert_permutation, expert_offset, expert_ids, workspace, st(stream));
}

int opmx_moe_select_index(const void *scores, int64_t T, int E, int k, int dtype, void *expert_weights,
                          int64_t *invert_permutation, int64_t *expert_offset, int32_t *row_token,
                          int32_t *expert_ids, void *workspace, size_t workspace_bytes, void *stream)
{
    if (T < 0 || E <= 0 || k <= 0 || k > E) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN)
        return OPMX_ERR_UNSUPPORTED;
    if (T > (int64_t{1} << 31) / k) return OPMX_ERR_UNSUPPORTED;
    if (!expert_offset) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!scores || !expert_weights || !invert_permutation || !row_token)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!workspace || workspace_bytes < moe_select_workspace_bytes(T, E, k))) return OPMX_ERR_WORKSPACE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OPMX_ERR_ALIGNMENT;
    return launch_moe_select(nullptr, scores, T, 0, E, k, dtype, nullptr, expert_weights, invert_permutation,
                             expert_offset, expert_ids, workspace, st(stream), row_token);
}

int opmx_moe_route_select_index(const void *X, const void *gate_weight, const void *gate_bias, int64_t T, int64_t H,
                                int E, int k, int dtype, void *scores, void *expert_weights,
                                int64_t *invert_permutation, int64_t *expert_offset, int32_t *row_token,
                                int32_t *expert_ids, void *workspace, size_t workspace_bytes, void *stream)
{
    if (T < 0 || H < 0 || E <= 0 || k <= 0 || k > E) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN)
        return OPMX_ERR_UNSUPPORTED;
    if (T > (int64_t{1} << 31) / k) return OPMX_ERR_UNSUPPORTED;
    if (!expert_offset) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!scores || !expert_weights || !invert_permutation || !row_token)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && H > 0 && (!X || !gate_weight)) return OPMX_ERR_BAD_ARGUMENT;
    if (T > 0 && (!workspace || workspace_bytes < moe_select_workspace_bytes(T, E, k))) return OPMX_ERR_WORKSPACE;
    if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u)) return OPMX_ERR_ALIGNMENT;
    return launch_moe_route_select(X, gate_weight, gate_bias, T, H, E, k, dtype, scores, nullptr, expert_weights,
                                   invert_permutation, expert_offset, expert_ids, workspace, st(stream), row_token);
}

size_t opmx_moe_grouped_gemm_workspace_bytes(int E, int64_t R, int64_t K, int64_t N, int dtype)
{
    return grouped_gemm_workspace_bytes(E, R, K, N, dtype);
}

static int grouped_checked(const void *X, const int64_t *off, const void *W, const void *B, int E, int64_t R,
                           int64_t K, int64_t N, int dtype, int epilogue, int64_t hint, void *Y, void *ws,
                           size_t ws_bytes, void *stream, RowGather g = {})
{
    if (E <= 0 || R < 0 || K < 0 || N < 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || E > OPMX_MOE_MAX_EXPERTS) return OPMX_ERR_UNSUPPORTED;
    if (epilogue != OPMX_EPILOGUE_NONE && epilogue != OPMX_EPILOGUE_SWIGLU) return OPMX_ERR_BAD_ARGUMENT;
    if (epilogue == OPMX_EPILOGUE_SWIGLU && N % 2) return OPMX_ERR_BAD_ARGUMENT;
    if (R == 0 || N == 0) return OPMX_OK;
    if (!X || !off || !W || !Y || K == 0) return OPMX_ERR_BAD_ARGUMENT;
    return launch_grouped_gemm(X, off, W, B, E, R, K, N, dtype, epilogue, hint, Y, ws, ws_bytes, st(stream), g);
}

int opmx_moe_column_parallel_linear(const void *X, const int64_t *expert_offset, const void *W, const void *B,
                                    int E, int64_t R, int64_t K, int64_t N, int dtype, int epilogue,
                                    int64_t rows_per_expert_hint, void *Y, void *workspace,
                                    size_t workspace_bytes, void *stream)
{
    return grouped_checked(X, expert_offset, W, B, E, R, K, N, dtype, epilogue, rows_per_expert_hint, Y,
                           workspace, workspace_bytes, stream);
}

int opmx_moe_column_parallel_linear_indexed(const void *X, int64_t X_rows, const int32_t *row_index,
                                            const int64_t *expert_offset, const void *W, const void *B, int E,
                                            int64_t R, int64_t K, int64_t N, int dtype, int epilogue,
                                            int64_t rows_per_expert_hint, void *Y, void *workspace,
                                            size_t workspace_bytes, void *stream)
{
    if (X_rows < 0 || (R > 0 && (X_rows == 0 || !row_index))) return OPMX_ERR_BAD_ARGUMENT;
    RowGather g;
    g.index = row_index;
    g.x_rows = X_rows;
    return grouped_checked(X, expert_offset, W, B, E, R, K, N, dtype, epilogue, rows_per_expert_hint, Y, workspace,
                           workspace_bytes, stream, g);
}

int opmx_moe_row_parallel_linear(const void *X, const int64_t *expert_offset, const void *W, const void *B,
                                 int E, int64_t R, int64_t K, int64_t N, int dtype,
                                 int64_t rows_per_expert_hint, void *Y, void *workspace, size_t workspace_bytes,
                                 void *stream)
{
    return grouped_checked(X, expert_offset, W, B, E, R, K, N, dtype, OPMX_EPILOGUE_NONE, rows_per_expert_hint,
                           Y, workspace, workspace_bytes, stream);
}

int opmx_swiglu(const void *X, int64_t R, int64_t D, float beta, int dtype, void *Y, void *stream)
{
    if (R < 0 || D < 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype)) return OPMX_ERR_UNSUPPORTED;
    if (R == 0 || D == 0) return OPMX_OK;
    if (!X || !Y) return OPMX_ERR_BAD_ARGUMENT;
    return launch_swiglu(X, R, D, beta, dtype, Y, st(stream));
}

int opmx_silu(const void *X, const void *gate, int64_t n, int dtype, void *Y, void *stream)
{
    if (n < 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype)) return OPMX_ERR_UNSUPPORTED;
    if (n == 0) return OPMX_OK;
    if (!X || !Y) return OPMX_ERR_BAD_ARGUMENT;
    return launch_silu(X, gate, n, dtype, Y, st(stream));
}

int opmx_rms_norm(const void *X, const void *weight, const void *SkipIn, int64_t T, int64_t H, float eps, int dtype,
                  void *Y, void *SkipOut, void *stream)
{
    if (T < 0 || H < 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype)) return OPMX_ERR_UNSUPPORTED;
    if (T > 0 && H > 0 && (!X || !weight || !Y)) return OPMX_ERR_BAD_ARGUMENT;
    if (!(eps >= 0.0f)) return OPMX_ERR_BAD_ARGUMENT;
    return launch_rms_norm(X, weight, SkipIn, T, H, eps, dtype, Y, SkipOut, st(stream));
}

int opmx_moe_reduce(const void *Y, const void *expert_weights, const int64_t *invert_permutation, int64_t T,
                    int k, int64_t N, int dtype, void *out, void *stream)
{
    if (T < 0 || N < 0 || k <= 0) return OPMX_ERR_BAD_ARGUMENT;
    if (!dtype_ok(dtype) || k > OPMX_MOE_MAX_EXPERTS_PER_TOKEN) return OPMX_ERR_UNSUPPORTED;
    if (T == 0 || N == 0) return OPMX_OK;
    if (!Y || !expert_weights || !invert_permutation || !out) return OPMX_ERR_BAD_ARGUMENT;
    return launch_moe_reduce(Y, expert_weights, invert_permutation, T, k, N, dtype, out, st(stream));
}

}  // extern "C"
