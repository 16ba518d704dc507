/*
 * opmx_moe.h - C ABI of libopmx_moe.so: the OPMX mixture-of-experts operators
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer on the GPU that is current on the
 *     calling thread; tensors are dense row-major; index tensors are int64,
 *     exactly like the reference operators' outputs;
 *   - `dtype` is an opmx_dtype value and applies to every floating tensor of
 *     the call (the reference operators are single-dtype too);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     all work is enqueued on it, nothing synchronises the device;
 *   - the library allocates nothing, frees nothing and keeps no pointer after
 *     a call returns; scratch memory comes in through `workspace` (the one
 *     exception, opmx_moe_select_static, says so below);
 *   - process-wide state, all of it thread-safe: (1) the first launch of a kernel
 *     on a GPU raises that kernel's shared-memory limit (hipFuncSetAttribute,
 *     remembered per GPU and kernel) -- make one call per shape outside a stream
 *     capture before capturing; (2) the compute-unit count of each GPU, looked up
 *     once; (3) the tuning knobs of opmx_moe_set_option, whose initial values are
 *     read once from the environment; (4) the per-GPU address of the scratch
 *     array of opmx_moe_select_static.  Calls on different streams or threads do
 *     not interfere as long as their buffers and workspaces differ;
 *   - every function returns OPMX_OK (0) or a negative opmx_status; on error
 *     nothing has been enqueued.  Faults inside a kernel surface, as with any
 *     HIP work, at the next synchronisation.
 *
 * The reference (OpenPPL/ppl.pmx) has no native interface: its operators are
 * torch.autograd.Function classes in torch_function/.  Each entry point below
 * names the Python function whose eager branch it replaces.
 */
#ifndef OPMX_MOE_H_
#define OPMX_MOE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OPMX_MOE_ABI_VERSION 1

typedef enum opmx_dtype {
    OPMX_DTYPE_F32 = 0,
    OPMX_DTYPE_F16 = 1,
    OPMX_DTYPE_BF16 = 2
} opmx_dtype;

typedef enum opmx_status {
    OPMX_OK = 0,
    OPMX_ERR_BAD_ARGUMENT = -1,   /* null pointer, negative size, k > E ...           */
    OPMX_ERR_UNSUPPORTED = -2,    /* dtype / E / k outside what the kernels cover      */
    OPMX_ERR_WORKSPACE = -3,      /* workspace missing or smaller than *_workspace_bytes */
    OPMX_ERR_ALIGNMENT = -4,      /* a pointer or row pitch is not aligned as required */
    OPMX_ERR_LAUNCH = -5          /* the HIP runtime refused a launch                  */
} opmx_status;

/* Epilogues of the grouped GEMM. */
typedef enum opmx_epilogue {
    OPMX_EPILOGUE_NONE = 0,
    /* Y[r, i] = H[r, D+i] * H[r, i] * sigmoid(H[r, i]) with H = X W^T (+B) and
     * D = N/2: SwiGLU (torch_function/SwiGLU.py:15-16, beta = 1) applied to the
     * fp32 accumulators; Y is [R, N/2]. */
    OPMX_EPILOGUE_SWIGLU = 1
} opmx_epilogue;

/* Limits of the routing kernels. */
#define OPMX_MOE_MAX_EXPERTS 256
#define OPMX_MOE_MAX_EXPERTS_PER_TOKEN 32

int opmx_moe_abi_version(void);
const char *opmx_status_string(int status);

/* Tuning / test knobs of the grouped GEMMs and the routing (no counterpart in the reference).  They choose
 * between kernels that compute the same thing; results change at most in accumulation order.
 * `name` is one of the strings below, `value` < 0 restores the automatic choice.  Each knob
 * starts from the environment variable of the same name, read once when the library is first
 * used (OPMX_MOE_GEMM accepts the words there).
 *   "OPMX_MOE_GEMM"                1 generic, 2 tiled, 3 stream: force a kernel family
 *   "OPMX_MOE_GEMM_TILED_VARIANT"  0 256x256 direct-to-LDS, 1 256x256 register-staged,
 *                                  2 128x128 register-staged, 3 128x256 direct-to-LDS
 *   "OPMX_MOE_GEMM_STREAM_VARIANT" 0..5: chunk widths / prefetch depth of the streaming kernel
 *   "OPMX_MOE_GEMM_GNX"            tile order: 8 expert-major, 16 row partition, 32 expert-grouped, 4, 0 row-major
 *   "OPMX_MOE_GEMM_STREAMK"        0 never split the tail tiles over K, 2 whenever possible
 *   "OPMX_MOE_GEMM_PERSIST"        0 never the persistent form, 1 whenever its conditions hold
 *   "OPMX_MOE_ROUTE_INDEX_TOKENS"  up to how many tokens (0 ... 64, then also up to 64 experts)
 *                                  opmx_moe_route_select_index runs as one launch of one block
 *   "OPMX_MOE_GEMM_F32_VARIANT"    float32 grouped GEMM: 0 the 128-column tile forms only, 1 always the
 *                                  32-row tiles whose waves split K
 * Returns OPMX_ERR_BAD_ARGUMENT for an unknown name. */
int opmx_moe_set_option(const char *name, int value);

/* Router gate / plain linear.  Replaces Linear.forward,
 * torch_function/Linear.py:25-33 (called from
 * model_zoo/mixtral/modeling/dynamic_batching/Model.py:188):
 *   Y[t, n] = sum_c X[t, c] * W[n, c] (+ B[n]),  fp32 accumulation.
 * X [T,K], W [N,K], B [N] or NULL, Y [T,N]. */
int opmx_linear(const void *X, const void *W, const void *B,
                int64_t T, int64_t K, int64_t N, int dtype, void *Y, void *stream);

/* MoeSelect.  Replaces MoeSelect.forward, torch_function/MoeSelect.py:37-64:
 * top-k of scores ordered (value desc, expert id asc), softmax over the k
 * picked values, stable sort of the T*k (token, slot) pairs by expert id.
 *   X [T,H], scores [T,E]                                     (dtype)
 *   X_expand_permute [T*k, H]                                 (dtype)
 *   expert_weights [T,k]                                      (dtype)
 *   invert_permutation [T*k] int64: row of X_expand_permute holding (t, slot)
 *   expert_offset [E+1] int64: rows of expert e are [off[e], off[e+1])
 * 1 <= k <= min(E, OPMX_MOE_MAX_EXPERTS_PER_TOKEN), E <= OPMX_MOE_MAX_EXPERTS.
 * expert_ids may be NULL; otherwise it receives the picked ids [T,k] as int32
 * (not an output of the reference operator; used by tests and fused callers). */
size_t opmx_moe_select_workspace_bytes(int64_t T, int E, int k);
int opmx_moe_select(const void *X, const void *scores, int64_t T, int64_t H, int E, int k,
                    int dtype, void *X_expand_permute, void *expert_weights,
                    int64_t *invert_permutation, int64_t *expert_offset, int32_t *expert_ids,
                    void *workspace, size_t workspace_bytes, void *stream);

/* MoeSelect for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference: it is
 * opmx_moe_select without the workspace argument, with the same inputs, outputs, limits and
 * results.  The scratch memory (chunk histograms and picked ids of calls with more than 256
 * tokens) is an array of OPMX_MOE_SELECT_STATIC_SCRATCH_BYTES bytes inside the library that
 * every GPU the library runs on holds until the process ends; the call allocates and frees
 * nothing.  A call whose opmx_moe_select_workspace_bytes(T, E, k) exceeds that size returns
 * OPMX_ERR_WORKSPACE (nothing enqueued).  All calls on one GPU share the array: two calls
 * that overlap on one GPU (different streams or threads) race; calls ordered on one stream
 * do not.  The first call on a GPU looks the array's address up and must be outside a
 * stream capture. */
#define OPMX_MOE_SELECT_STATIC_SCRATCH_BYTES (4u << 20)
int opmx_moe_select_static(const void *X, const void *scores, int64_t T, int64_t H, int E, int k,
                           int dtype, void *X_expand_permute, void *expert_weights,
                           int64_t *invert_permutation, int64_t *expert_offset, int32_t *expert_ids,
                           void *stream);

/* Router gate and MoeSelect in one call: scores = X gate_weight^T (+ gate_bias), then
 * opmx_moe_select on those scores.  Replaces the pair of calls at
 * model_zoo/mixtral/modeling/dynamic_batching/Model.py:188-190 (self.gate, then
 * OPMX.moe_select); the two operators stay callable on their own.
 *   X [T,H], gate_weight [E,H], gate_bias [E] or NULL          (dtype)
 *   scores [T,E]: receives the router logits (an input of opmx_moe_select, an output here)
 *   the other outputs, the limits and the workspace are those of opmx_moe_select.
 * Three regimes (fp16/bf16 with H % 32 == 0 and 16-byte aligned X / gate_weight; anything else, and
 * float32, runs opmx_linear and opmx_moe_select one after the other):
 *   T <= 8 and E <= 16   one launch: every block recomputes the few logits on the MFMA units, routes
 *                        all tokens and emits its own token's outputs (the index form,
 *                        opmx_moe_route_select_index, has no row copies to spread over blocks and
 *                        runs as one block that does everything);
 *   T > 256 and E <= 64  where the K-split MFMA router kernel serves the shape (see opmx_linear), it
 *                        routes its 16 tokens per block in its epilogue -- top-k and softmax on the
 *                        rounded logits it has just written -- and MoeSelect starts from the picks
 *                        (histogram, scan, rank, row copies): one launch and the read-back of the
 *                        logits less;
 *   otherwise            the router kernel, then the MoeSelect kernels (a dependent launch costs
 *                        about 4 us on this device; one block computing the logits of more than a
 *                        handful of tokens costs more: a CU's load path moves 64 bytes per clock).
 * Routing is exact on the returned scores in every regime; the scores themselves may differ from
 * opmx_linear's in the last bit (other summation order of the fp32 accumulation). */
int opmx_moe_route_select(const void *X, const void *gate_weight, const void *gate_bias, int64_t T,
                          int64_t H, int E, int k, int dtype, void *scores, void *X_expand_permute,
                          void *expert_weights, int64_t *invert_permutation, int64_t *expert_offset,
                          int32_t *expert_ids, void *workspace, size_t workspace_bytes, void *stream);

/* MoeSelect without the row copy (torch_function/MoeSelect.py:37-64 except :45-47): the routing
 * outputs of opmx_moe_select -- expert_weights, invert_permutation, expert_offset, bit for bit
 * the same -- and, instead of X_expand_permute, the index that stands for it:
 *   row_token [T*k] int32: row r of X_expand_permute would be X[row_token[r], :]
 *                          (row_token[invert_permutation[t*k+s]] = t; perm[r] / k in the reference's terms).
 * opmx_moe_column_parallel_linear_indexed reads X through it, so the [T*k, H] copy is never
 * written or read.  Limits and workspace are those of opmx_moe_select.
 * opmx_moe_route_select_index is the same with the router gate in front (see
 * opmx_moe_route_select): scores [T,E] is then an output. */
int opmx_moe_select_index(const void *scores, int64_t T, int E, int k, int dtype, void *expert_weights,
                          int64_t *invert_permutation, int64_t *expert_offset, int32_t *row_token,
                          int32_t *expert_ids, void *workspace, size_t workspace_bytes, void *stream);
int opmx_moe_route_select_index(const void *X, const void *gate_weight, const void *gate_bias, int64_t T,
                                int64_t H, int E, int k, int dtype, void *scores, void *expert_weights,
                                int64_t *invert_permutation, int64_t *expert_offset, int32_t *row_token,
                                int32_t *expert_ids, void *workspace, size_t workspace_bytes, void *stream);

/* Grouped expert GEMM.  Replaces the per-expert F.linear loops of
 * MoeColumnParallelLinear.forward (torch_function/MoeColumnParallelLinear.py:58-69)
 * and MoeRowParallelLinear.forward (torch_function/MoeRowParallelLinear.py:44-60)
 * at tensor-parallel world size 1:
 *   for e in [0,E), r in [off[e], off[e+1]):  Y[r,:] = X[r,:] W[e]^T (+ B[e])
 * rows outside [off[0], off[E]) are set to zero.  expert_offset is read on the
 * device; it must be non-decreasing with values in [0, R].
 *   X [R,K], W [E,N,K], B [E,N] or NULL, Y [R,N] (or [R,N/2] with the SwiGLU epilogue).
 * float16 / bfloat16 run on the fp16 / bf16 matrix units (weight-streaming kernel for few rows
 * per expert, tile kernels beyond), float32 on the fp32 matrix units (K % 4 == 0, 16-byte aligned
 * X and W); every other shape takes a shape-agnostic kernel.  Accumulation is fp32 throughout.
 * `rows_per_expert_hint` is the largest segment the caller can guarantee
 * (for MoeSelect output: min(R, T)); 0 = unknown.  It only selects between
 * kernel variants, never correctness.
 * `workspace` is optional scratch memory (16-byte aligned device memory of at least
 * opmx_moe_grouped_gemm_workspace_bytes() bytes, contents arbitrary, not shared with a
 * call running at the same time): with it the large-tile kernel cuts the tiles of its
 * last, partly filled round into k-ranges that run side by side and meet in fp32 in the
 * workspace (down projections with few tiles and a long K gain 7-13 %).  NULL / 0 is
 * always accepted; the result is then accumulated in a single pass per tile. */
size_t opmx_moe_grouped_gemm_workspace_bytes(int E, int64_t R, int64_t K, int64_t N, int dtype);
int opmx_moe_column_parallel_linear(const void *X, const int64_t *expert_offset, const void *W,
                                    const void *B, int E, int64_t R, int64_t K, int64_t N,
                                    int dtype, int epilogue, int64_t rows_per_expert_hint,
                                    void *Y, void *workspace, size_t workspace_bytes, void *stream);
/* opmx_moe_column_parallel_linear with its rows read through an index: GEMM row r is
 * X[row_index[r], :] with X [X_rows, K] (the tokens, not their expanded copies) and row_index
 * [R] int32 with values in [0, X_rows) -- the row_token output of opmx_moe_select_index.  Equals
 * opmx_moe_column_parallel_linear on X_expand_permute bit for bit (the reference gathers first,
 * torch_function/MoeSelect.py:45-47, then multiplies, MoeColumnParallelLinear.py:58-67).
 * fp16 / bf16 kernels need X_rows * K * 2 < 2^31 (else the shape-agnostic fallback kernel runs). */
int opmx_moe_column_parallel_linear_indexed(const void *X, int64_t X_rows, const int32_t *row_index,
                                            const int64_t *expert_offset, const void *W, const void *B, int E,
                                            int64_t R, int64_t K, int64_t N, int dtype, int epilogue,
                                            int64_t rows_per_expert_hint, void *Y, void *workspace,
                                            size_t workspace_bytes, void *stream);
int opmx_moe_row_parallel_linear(const void *X, const int64_t *expert_offset, const void *W,
                                 const void *B, int E, int64_t R, int64_t K, int64_t N,
                                 int dtype, int64_t rows_per_expert_hint,
                                 void *Y, void *workspace, size_t workspace_bytes, void *stream);

/* SwiGLU.  Replaces SwiGLU.forward, torch_function/SwiGLU.py:11-17:
 *   Y[r, i] = X[r, D+i] * X[r, i] * sigmoid(beta * X[r, i]);  X [R,2D], Y [R,D]. */
int opmx_swiglu(const void *X, int64_t R, int64_t D, float beta, int dtype, void *Y, void *stream);

/* Gated SiLU.  Replaces SiLU.forward, torch_function/SiLU.py:14-21:
 *   Y[i] = gate[i] * X[i] * sigmoid(X[i])  (gate may be NULL);  n elements. */
int opmx_silu(const void *X, const void *gate, int64_t n, int dtype, void *Y, void *stream);

/* RMSNorm / SkipRMSNorm over the last dimension: the operator in front of the MoE layer
 * (ffn_norm, model_zoo/mixtral/modeling/dynamic_batching/Model.py:261).  Replaces
 * RMSNorm.forward and SkipRMSNorm.forward, torch_function/RMSNorm.py:16-24 and :44-56:
 *   s = X + SkipIn (rounded to dtype; s = X when SkipIn is NULL)
 *   Y = round(round(s * rsqrt(mean(s^2) + eps)) * weight),  SkipOut = s
 * X, SkipIn, Y, SkipOut [T,H]; weight [H]; SkipOut may be NULL (plain RMSNorm). */
int opmx_rms_norm(const void *X, const void *weight, const void *SkipIn, int64_t T, int64_t H, float eps,
                  int dtype, void *Y, void *SkipOut, void *stream);

/* MoeReduce.  Replaces MoeReduce.forward, torch_function/MoeReduce.py:16-26:
 *   out[t, :] = sum_{s<k} expert_weights[t,s] * Y[invert_permutation[t*k+s], :]
 * summed in slot order in fp32, rounded once.  Y [T*k,N], out [T,N].
 * invert_permutation values must lie in [0, T*k). */
int opmx_moe_reduce(const void *Y, const void *expert_weights, const int64_t *invert_permutation,
                    int64_t T, int k, int64_t N, int dtype, void *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* OPMX_MOE_H_ */
