/*
 * moe355.h -- C ABI of libmoe355.so: the W8A8-dynamic fused-MoE layer of
 * vllm-ascend as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says "host";
 *   - every call only enqueues work on `stream` (a hipStream_t passed as void*)
 *     and returns; it never synchronises, allocates or frees;
 *   - scratch memory comes from the caller: ask moe355_*_workspace() for the
 *     byte count, pass a 256-byte aligned buffer of at least that size
 *     (one entry point keeps its scratch in a fixed device array instead and says so:
 *     moe355_init_routing_static);
 *   - return value 0 = enqueued; negative = rejected, nothing was enqueued
 *     (see MOE355_E_*; moe355_strerror() gives the text);
 *   - tensors are dense row-major; "bf16" means raw bfloat16 bits.  Wherever hidden states are bf16 they may
 *     also be fp16 (MOE355_DT_F16 in the dtype argument), the model dtype of the reference: the same arithmetic
 *     in fp32, narrowed to fp16 by round-to-nearest-even at the points where the text says bf16;
 *   - `dtype` arguments use MOE355_DT_*.
 *
 * Each entry point names the interface of the reference tree (vllm-ascend,
 * paths relative to its root) that it stands in for.
 */
#ifndef MOE355_H
#define MOE355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE355_ABI_VERSION 1

enum {
    MOE355_OK = 0,
    MOE355_E_ARG = -1,       /* null pointer, negative size, unknown enum value */
    MOE355_E_SHAPE = -2,     /* shape outside what the kernels support (alignment, limits) */
    MOE355_E_WORKSPACE = -3, /* workspace missing, misaligned or too small */
    MOE355_E_LAUNCH = -4,    /* the HIP runtime refused the launch */
    MOE355_E_UNSUPPORTED = -5
};

enum { MOE355_DT_F32 = 0, MOE355_DT_BF16 = 1, MOE355_DT_F16 = 2 };

/* layouts accepted by moe355_format_cast_nz */
enum {
    MOE355_W_ENK = 0, /* [E, N, K]: one row of K per output channel (checkpoint order) */
    MOE355_W_EKN = 1  /* [E, K, N]: the order the reference holds after its transpose
                         (vllm_ascend/quantization/methods/w8a8_dynamic.py:346-347) */
};

/* meaning of a group list, as in the reference (vllm_ascend/ops/fused_moe/moe_mlp.py:54-83) */
enum { MOE355_GL_CUMSUM = 0, MOE355_GL_COUNT = 1 };

int moe355_abi_version(void);
const char *moe355_strerror(int code);

/* ---------------------------------------------------------------------------
 * Per-token dynamic int8 quantisation.
 * Stands in for torch_npu.npu_dynamic_quant as called from
 * vllm_ascend/device/device_op.py:192-206 (moe_mlp.py:237-242) and the shared
 * expert (vllm_ascend/ops/fused_moe/shared_experts.py:258).
 *   a = max|row| ; scale = a/127 ; q = clamp(rint(v/scale), -128, 127) ; a == 0 -> q = 0, scale = 0
 * x [rows, cols] bf16 / fp16 -> q [rows, cols] int8, scale [rows] fp32.
 */
int moe355_dynamic_quant(const void *x, int x_dtype, int64_t rows, int64_t cols, int8_t *q, float *scale,
                         void *stream);

/* The same operator with the division chosen by the caller.  form 0: what moe355_dynamic_quant and every other
 * token quantiser of this library run (one reciprocal per row, the product corrected once; rows whose scale lies
 * outside [2^-100, 2^100] divide); form 1: the general IEEE division on every value, which is the definition above.
 * No operator of the reference stands behind it: a bf16 / fp16 row holds values of 2^16 patterns below a maximum
 * of 2^15, so a test can run every (maximum, value) pair through both forms and find the same int8. */
int moe355_dynamic_quant_form(const void *x, int x_dtype, int64_t rows, int64_t cols, int8_t *q, float *scale,
                              int form, void *stream);

/* ---------------------------------------------------------------------------
 * Router gate: logits = x.float() @ weight.T (+ bias) in fp32.
 * Stands in for AscendGateLinear.forward (vllm_ascend/ops/fused_moe/gate_linear.py:55-63) and the
 * internal-router branch of the layer (vllm_ascend/ops/fused_moe/fused_moe.py:264-271), both of which end in
 * F.linear on fp32 operands.  Summation order (the reference leaves it to its BLAS): K in chunks of 128, a
 * fused multiply-add chain over ascending k from +0 inside a chunk, chunk results added in ascending order to
 * a total that starts at +0, bias last.
 * x [T, hidden] bf16, fp16 or fp32; weight [E, hidden] fp32; bias [E] fp32 or NULL -> logits [T, E] fp32.
 * hidden must be a multiple of 64 and below 2^22, num_experts * hidden below 2^30 (MOE355_E_SHAPE otherwise).
 * Few tokens (fewer than 192 output tiles of 32 x 32) run one workgroup per K chunk and need the workspace
 * (256-byte aligned); otherwise the workspace size is 0 and it may be NULL.
 */
size_t moe355_router_gate_workspace(int64_t num_tokens, int hidden, int num_experts);
int moe355_router_gate(const void *x, int x_dtype, const float *weight, const float *bias, int64_t num_tokens,
                       int hidden, int num_experts, float *logits, void *workspace, size_t workspace_bytes,
                       void *stream);

/* ---------------------------------------------------------------------------
 * Group-limited top-k gating.
 * Stands in for aclnnMoeGatingTopK behind torch.ops._C_ascend.moe_gating_top_k
 * (csrc/moe/moe_gating_top_k/moe_gating_top_k_torch_adpt.h:19-71, schema
 * csrc/torch_binding.cpp:2135-2150).  Argument meaning is the reference's:
 * norm_type 0 softmax / 1 sigmoid; group_select_mode 0 max / 1 sum of top-2;
 * bias is used for selection only; renorm or sigmoid divides by (sum + eps).
 * x [rows, E] (x_dtype), bias [E] (x_dtype) or NULL ->
 * y [rows, k] (x_dtype), expert_idx [rows, k] int32, out [rows, E] fp32
 * (written only when out_flag != 0; may be NULL otherwise).
 * y_alt (optional, NULL to skip): a second copy of y, narrowed from the value stored
 * in y to y_alt_dtype -- the cast the reference's caller applies next
 * (topk_weights.to(hidden dtype), vllm_ascend/ops/fused_moe/routed_experts.py:482).
 * Limits: E <= 2048, k <= 64, group_count <= 64.
 */
int moe355_gating_top_k(const void *x, int x_dtype, const void *bias, int64_t rows, int64_t num_experts, int k,
                        int k_group, int group_count, int group_select_mode, int renorm, int norm_type, int out_flag,
                        float routed_scaling_factor, float eps, void *y, int32_t *expert_idx, float *out,
                        void *y_alt, int y_alt_dtype, void *stream);

/* ---------------------------------------------------------------------------
 * Expert histogram + stable counting sort of the flattened [T*k] expert ids +
 * token gather with fused per-row int8 quantisation.
 * Stands in for torch_npu.npu_moe_init_routing_v2 as called from
 * vllm_ascend/device/device_op.py:103-127 (token_dispatcher.py:424-435):
 *   expanded_row_idx[t*k+j] = row of pair (t, j) in the expert-sorted array,
 *   the sort being stable in the flat index (vllm_ascend/lora/fused_moe.py:190-204).
 * quant_mode 1: expanded_x is int8 [R, H] and dynamic_scale [R] fp32 is written;
 * quant_mode -1: expanded_x is a [R, H] copy in x's dtype and dynamic_scale is ignored.
 * expert_tokens [E] int64: per-expert counts (tokens_num_type 1) or their
 * running sum (tokens_num_type 0).
 * x [T, H] bf16 / fp16, expert_idx [T, k] int32 in [0, E).  A pair whose id lies outside the range is
 * dropped: it is not counted, takes no row, and its expanded_row_idx is R = T*k, one past the last row --
 * an index that moe355_token_unpermute skips (and that survives the abs() the reference's caller applies,
 * vllm_ascend/device/device_op.py:950-954).  Rows of expanded_x past the last valid pair are left untouched.
 * R must be < 2^31.
 */
size_t moe355_init_routing_workspace(int64_t num_tokens, int top_k, int num_experts);
int moe355_init_routing(const void *x, int x_dtype, int64_t num_tokens, int64_t hidden, const int32_t *expert_idx,
                        int top_k, int num_experts, int quant_mode, int tokens_num_type, void *expanded_x,
                        int32_t *expanded_row_idx, int64_t *expert_tokens, float *dynamic_scale, void *workspace,
                        size_t workspace_bytes, void *stream);

/* The maps of the permutation alone, nothing moved: expanded_row_idx [T*k] (pair -> sorted row, T*k for a
 * dropped pair), row_token [T*k] (sorted row -> token; entries past the last kept pair are left untouched) and
 * expert_tokens, exactly as moe355_init_routing computes them.  For callers that quantise the token rows once
 * (moe355_dynamic_quant) and let moe355_gmm1_swiglu_quant_gather read them through row_token instead of
 * writing k copies of every row: no counterpart of its own in the reference, it is the index half of
 * torch_npu.npu_moe_init_routing_v2 (vllm_ascend/ops/fused_moe/token_dispatcher.py:424-435).  The workspace is
 * the one of moe355_init_routing_workspace. */
int moe355_route_map(const int32_t *expert_idx, int64_t num_tokens, int top_k, int num_experts, int tokens_num_type,
                     int32_t *expanded_row_idx, int32_t *row_token, int64_t *expert_tokens, void *workspace,
                     size_t workspace_bytes, void *stream);

/* The same permutation for activations that are already quantised: x int8 [T, H] with one fp32 scale per
 * token; rows and scales are only moved (expanded_x[row] = x[t], expanded_scale[row] = x_scale[t]).
 * Stands in for torch_npu.npu_moe_init_routing_v2(x, ids, scale=pertoken_scale, quant_mode=-1), the call the
 * dispatcher makes when the layer was handed pre-quantised hidden states
 * (vllm_ascend/ops/fused_moe/token_dispatcher.py:399-435 with routing.pertoken_scale set; the expert MLP then
 * skips its own quantisation, vllm_ascend/ops/fused_moe/moe_mlp.py:226-242).  H % 16 == 0; the workspace is
 * the one of moe355_init_routing_workspace. */
int moe355_init_routing_prequant(const int8_t *x, const float *x_scale, int64_t num_tokens, int64_t hidden,
                                 const int32_t *expert_idx, int top_k, int num_experts, int tokens_num_type,
                                 int8_t *expanded_x, int32_t *expanded_row_idx, int64_t *expert_tokens,
                                 float *expanded_scale, void *workspace, size_t workspace_bytes, void *stream);

/* moe355_init_routing without a workspace argument: for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid allocation).  No counterpart in the reference.
 * The scratch of the routing kernels (chunk histograms, expert offsets, partition bases) lives in a fixed
 * device array of MOE355_INIT_ROUTING_STATIC_BYTES that every GPU the library runs on holds until the process
 * ends; its address is looked up once per device, on the first call with that device current.  The call itself
 * allocates and frees nothing.  Batches whose scratch (moe355_init_routing_workspace) does not fit the array are
 * rejected with MOE355_E_WORKSPACE.  All calls on one GPU share the array: calls that overlap in time on one
 * GPU (different streams, different threads) race and must be serialised by the caller.  The address is cached
 * for the device that is current at the call, which must be the device that owns `stream`; the first call on a
 * device does that lookup (host-side runtime work) and must therefore be made outside stream capture.  Results
 * are identical to moe355_init_routing's. */
#define MOE355_INIT_ROUTING_STATIC_BYTES (2u << 20)
int moe355_init_routing_static(const void *x, int x_dtype, int64_t num_tokens, int64_t hidden,
                               const int32_t *expert_idx, int top_k, int num_experts, int quant_mode,
                               int tokens_num_type, void *expanded_x, int32_t *expanded_row_idx,
                               int64_t *expert_tokens, float *dynamic_scale, void *stream);

/* ---------------------------------------------------------------------------
 * Small batches (decode): the gating op and the init-routing op in ONE launch.
 * No single counterpart in the reference: it stands in for the pair
 *   torch.ops._C_ascend.moe_gating_top_k (vllm_ascend/ops/fused_moe/router/fused_topk_router.py:84-159) +
 *   torch_npu.npu_moe_init_routing_v2(quant_mode=1) (vllm_ascend/ops/fused_moe/token_dispatcher.py:424-435)
 * with the arithmetic of moe355_gating_top_k and moe355_init_routing, for batches of at most 1024 (token, slot)
 * pairs over at most 256 experts (moe355_route_quant_small_supported() != 0), where two launches of a few
 * microseconds each are a visible part of the layer.  Some workgroups gate four tokens each and the last of
 * them to finish sorts the pairs (nobody waits); the others quantise one token row each.
 * The int8 rows are written ONCE, in token order: row r of the expert-sorted
 * activation is xq[row_token[r]] with scale x_scale[row_token[r]], which is how moe355_gmm1_swiglu_quant_gather
 * reads it; nothing is copied k times.
 *   logits [T, E] (logits_dtype), bias [E] (logits_dtype) or NULL, x [T, H] bf16 / fp16 ->
 *   topk_weights [T, k] in x's dtype (the gate's weights rounded to the logits dtype, then to x's dtype),
 *   topk_ids [T, k] int32, xq [T, H] int8, x_scale [T] fp32, expanded_row_idx [T*k] int32,
 *   row_token [T*k] int32, expert_tokens [E] int64 (counts, or their running sum for tokens_num_type 0).
 * sync_counter: ONE int32 in device memory that is 0 when the call starts to execute; the call leaves it at 0.
 * (Allocate it once, zeroed, and keep it; calls that may overlap in time need counters of their own.)
 */
int moe355_route_quant_small_supported(int64_t num_tokens, int top_k, int num_experts);
int moe355_route_quant_small(const void *x, int x_dtype, const void *logits, int logits_dtype, const void *bias,
                             int64_t num_tokens, int64_t hidden, int num_experts, int k, int k_group,
                             int group_count, int group_select_mode, int renorm, int norm_type,
                             float routed_scaling_factor, float eps, int tokens_num_type, void *topk_weights,
                             int32_t *topk_ids, int8_t *xq, float *x_scale, int32_t *expanded_row_idx,
                             int32_t *row_token, int64_t *expert_tokens, int32_t *sync_counter, void *stream);

/* Gating and token quantisation in one launch, for any number of tokens (at most 256 experts:
 * moe355_gate_quant_supported() != 0): the two steps read different inputs, so their workgroups run side by side.
 * Stands in for the pair torch.ops._C_ascend.moe_gating_top_k
 * (vllm_ascend/ops/fused_moe/router/fused_topk_router.py:84-159) + the per-token quantisation inside
 * torch_npu.npu_moe_init_routing_v2(quant_mode=1) (vllm_ascend/ops/fused_moe/token_dispatcher.py:424-435), with
 * the arithmetic of moe355_gating_top_k and moe355_dynamic_quant; moe355_route_map then builds the index maps.
 * Outputs as in moe355_route_quant_small: topk_weights [T, k] in x's dtype, topk_ids [T, k], xq [T, H] int8,
 * x_scale [T]. */
int moe355_gate_quant_supported(int64_t num_tokens, int top_k, int num_experts);
int moe355_gate_quant(const void *x, int x_dtype, const void *logits, int logits_dtype, const void *bias,
                      int64_t num_tokens, int64_t hidden, int num_experts, int k, int k_group, int group_count,
                      int group_select_mode, int renorm, int norm_type, float routed_scaling_factor, float eps,
                      void *topk_weights, int32_t *topk_ids, int8_t *xq, float *x_scale, void *stream);

/* ---------------------------------------------------------------------------
 * Weight format cast: dense int8 weights -> the MFMA-tiled storage the grouped
 * GEMMs stream ("NZ" of this build).  Stands in for
 * torch_npu.npu_format_cast(w, ACL_FORMAT_FRACTAL_NZ) in
 * vllm_ascend/quantization/methods/w8a8_dynamic.py:350-351.
 * Tiled storage: [E][N/32][K/32][64][16] bytes; inside a 1 KiB tile, entry
 * (lane, b) holds w[e, 32*nb + lane%32, 32*kb + 16*(lane/32) + b].
 * N and K must be multiples of 32.  out has E*N*K bytes and must not alias w.
 */
int moe355_format_cast_nz(const int8_t *w, int layout, int64_t num_experts, int64_t n, int64_t k, int8_t *out,
                          void *stream);

/* int4 weights (W4A8): two 4-bit two's-complement values per byte.
 * source 0: w is int8 [E, N, K] holding one int4 value (-8..7) per byte (checkpoint order);
 * source 1: w is packed [E, K, N/2] bytes, low nibble = even channel, the packing of
 *           vllm_ascend/quantization/methods/w4a8.py:327-336.
 * out: tiled int4 storage, E*N*K/2 bytes: [E][N/32][K/64][64][16]; inside a 1 KiB tile, byte b of
 * entry `lane` holds w[e, 32*nb + lane%32, 64*kb + 16*(lane/32) + b] in its low nibble and the
 * value 32 further along K in its high nibble.  N % 32 == 0, K % 64 == 0. */
int moe355_format_cast_nz_int4(const uint8_t *w, int source, int64_t num_experts, int64_t n, int64_t k, uint8_t *out,
                               void *stream);

/* ---------------------------------------------------------------------------
 * gate_up grouped GEMM (int8 x int8 -> int32) + dequant + SwiGLU + per-row int8
 * re-quantisation.
 * Stands in for aclnnGroupedMatmulSwigluQuantWeightNZ behind
 * torch.ops._C_ascend.grouped_matmul_swiglu_quant_weight_nz
 * (csrc/gmm/grouped_matmul_swiglu_quant_weight_nz_tensor_list/grouped_matmul_swiglu_quant_torch_adpt.h:20-51,
 * schema csrc/torch_binding.cpp:2025-2037; math
 * csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:370-522):
 *   f = (float(acc) * x_scale[row]) * weight_scale[e, col]
 *   y = silu(f[:, :N/2]) * f[:, N/2:] ; out_scale = max|y|/127 ; out = rint(y * (1/out_scale))
 * x [R, K] int8; weight: tiled storage of [E, N, K] (moe355_format_cast_nz);
 * weight_scale [E, N] fp32; x_scale [R] fp32; group_list [E] int64
 * (group_list_type MOE355_GL_*); out [R, N/2] int8; out_scale [R] fp32.
 * Rows at or beyond the last cumulative count are left untouched.
 * swiglu_limit > 0 clamps gate to <= L and up to [-L, L].
 * Limits: N % 64 == 0, K % 32 == 0.
 */
size_t moe355_gmm1_swiglu_quant_workspace(int64_t rows, int64_t n, int64_t k, int num_experts);
int moe355_gmm1_swiglu_quant(const int8_t *x, const int8_t *weight_nz, const float *weight_scale,
                             const float *x_scale, const int64_t *group_list, int group_list_type, int64_t rows,
                             int64_t k, int64_t n, int num_experts, float swiglu_limit, int8_t *out,
                             float *out_scale, void *workspace, size_t workspace_bytes, void *stream);

/* The same op on activations that were quantised in token order and not gathered (moe355_route_quant_small, or
 * moe355_dynamic_quant + moe355_route_map): x [T, K] int8, x_scale [T]; row r of the expert-sorted order is
 * x[row_token[r]] with scale x_scale[row_token[r]] (row_token [rows] int32).  out / out_scale are in the
 * expert-sorted order, as above.  Every kernel family reads its token rows through the map. */
int moe355_gmm1_swiglu_quant_gather(const int8_t *x, const float *x_scale, const int32_t *row_token,
                                    const int8_t *weight_nz, const float *weight_scale, const int64_t *group_list,
                                    int group_list_type, int64_t rows, int64_t k, int64_t n, int num_experts,
                                    float swiglu_limit, int8_t *out, float *out_scale, void *workspace,
                                    size_t workspace_bytes, void *stream);

/* Per-expert tensors: weight_nz_list / weight_scale_list are DEVICE arrays of num_experts pointers,
 * entry e pointing at expert e's tiled [N, K] weights / its [N] fp32 scales (experts that can be
 * swapped one by one, as dynamic expert load balancing does).  Stands in for
 * torch.ops._C_ascend.grouped_matmul_swiglu_quant_weight_nz_tensor_list (csrc/torch_binding.cpp:2039-2045). */
int moe355_gmm1_swiglu_quant_list(const int8_t *x, const int8_t *const *weight_nz_list,
                                  const float *const *weight_scale_list, const float *x_scale,
                                  const int64_t *group_list, int group_list_type, int64_t rows, int64_t k, int64_t n,
                                  int num_experts, float swiglu_limit, int8_t *out, float *out_scale, void *workspace,
                                  size_t workspace_bytes, void *stream);

/* W4A8 variant: int4 weights (moe355_format_cast_nz_int4 storage), fp32 scales per group of
 * `group_size` values along K: weight_scale [E, K/group_size, N] (group_size == K: per channel).
 *   f = (sum_g float(acc_g) * weight_scale[e, g, col] (g ascending) + bias[e, col]) * x_scale[row]
 * then SwiGLU and re-quantisation as above.  bias [E, N] fp32 or NULL.
 * Stands in for the int4 form of torch.ops._C_ascend.grouped_matmul_swiglu_quant /
 * grouped_matmul_swiglu_quant_v2 (csrc/torch_binding.cpp:2025-2053; kernel
 * csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant_a8w4_msd_*.h; golden
 * tests/e2e/nightly/single_node/ops/singlecard_ops/test_grouped_matmul_swiglu_quant.py:22-109).
 * Workspace: rows * (n/2) * 4 bytes.  Limits: N % 64 == 0, K % 64 == 0, group_size % 64 == 0. */
int moe355_gmm1_swiglu_quant_w4(const int8_t *x, const uint8_t *weight_nz4, const float *weight_scale,
                                int64_t group_size, const float *bias, const float *x_scale,
                                const int64_t *group_list, int group_list_type, int64_t rows, int64_t k, int64_t n,
                                int num_experts, float swiglu_limit, int8_t *out, float *out_scale, void *workspace,
                                size_t workspace_bytes, void *stream);

/* corr[e, col] = 8 * sum_g float(sum_{k in g} w[e, col, k]) * weight_scale[e, g, col]  (fp32 [E, N]).
 * The reference's int4 op computes (x - 8) . W and expects the caller to pass this term back in as
 * `bias` / `weight_assist_matrix` (vllm_ascend/quantization/methods/w4a8.py:385-394); a caller of
 * moe355_gmm1_swiglu_quant_w4, which computes x . W, passes `bias - corr` instead. */
int moe355_w4_offset_correction(const uint8_t *weight_nz4, const float *weight_scale, int64_t group_size,
                                int num_experts, int64_t n, int64_t k, float *corr, void *stream);

/* Activations other than SiLU between the two grouped GEMMs.  Stands in for the unfused branch of
 * quant_apply_mlp (vllm_ascend/ops/fused_moe/moe_mlp.py:484-549): the gate_up product is dequantised to the hidden
 * dtype (moe355_gmm2_dequant with the gate_up weights), then this call applies the activation and the dynamic
 * quantiser (torch_npu.npu_dynamic_quant) in one pass:
 *   MOE355_ACT_GELU / _GELU_TANH  gelu(gate) * up                                  (moe_mlp.py:516-520)
 *   MOE355_ACT_SWIGLUSTEP         min(silu(gate), L) * clamp(up, -L, L), L = limit > 0   (moe_mlp.py:512-515)
 *   MOE355_ACT_SWIGLUOAI          g = min(gate, L), u = clamp(up, -L, L) (L = limit, 0: no clamp):
 *                                 g * sigmoid(alpha * g) * (u + beta)                (moe_mlp.py:123-137, 521-538)
 * evaluated in fp32 on the 16-bit inputs, rounded once to the 16-bit dtype, then scale = absmax / 127,
 * q = rint(v / scale).  h [rows, n] bf16 / fp16 (gate = first n/2 columns); q [rows, n/2] int8; scale [rows].
 * group_list (optional): rows at or beyond its total are left untouched. */
enum { MOE355_ACT_GELU = 1, MOE355_ACT_GELU_TANH = 2, MOE355_ACT_SWIGLUSTEP = 3, MOE355_ACT_SWIGLUOAI = 4 };
int moe355_act_mul_quant(const void *h, int h_dtype, const int64_t *group_list, int group_list_type, int num_experts,
                         int64_t rows, int64_t n, int activation, float limit, float alpha, float beta, int8_t *q,
                         float *scale, void *stream);

/* The gate function of the SwiGLU epilogues by itself: out[i] = g[i] / (1 + exp(-g[i])) in fp32, n values.
 * form 0: the instruction sequence every kernel of this library runs (a division specialised to a divisor in
 * [1, 2^128)); form 1: the same function with the general IEEE division, which is the definition
 * (csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:461-485,
 * csrc/gmm/grouped_matmul_swiglu_quant/README.md:63-67) and what the CPU checker computes.  No operator of the
 * reference stands behind it: it exists so that a test can run both forms over all 2^32 inputs and find them
 * equal bit for bit. */
int moe355_silu_f32(const float *g, float *out, int64_t n, int form, void *stream);

/* ---------------------------------------------------------------------------
 * down grouped GEMM (int8 x int8 -> int32) + dequant to bf16.
 * Stands in for torch_npu.npu_grouped_matmul(scale=, per_token_scale=,
 * group_type=0, split_item=2) as called from vllm_ascend/device/device_op.py:254-291:
 *   out[row, col] = bf16( (float(acc) * per_token_scale[row]) * scale[e, col] )
 * x [R, K] int8; weight tiled [E, N, K]; scale [E, N] fp32; out [R, N] bf16 or fp16 (out_dtype).
 */
size_t moe355_gmm2_dequant_workspace(int64_t rows, int64_t n, int64_t k, int num_experts);
int moe355_gmm2_dequant(const int8_t *x, const int8_t *weight_nz, const float *scale, const float *per_token_scale,
                        const int64_t *group_list, int group_list_type, int64_t rows, int64_t k, int64_t n,
                        int num_experts, void *out, int out_dtype, void *workspace, size_t workspace_bytes,
                        void *stream);

/* Per-expert tensor form of the down projection (weight list of torch_npu.npu_grouped_matmul,
 * vllm_ascend/device/device_op.py:280-291 with `weight` a list of E tensors). */
int moe355_gmm2_dequant_list(const int8_t *x, const int8_t *const *weight_nz_list, const float *const *scale_list,
                             const float *per_token_scale, const int64_t *group_list, int group_list_type,
                             int64_t rows, int64_t k, int64_t n, int num_experts, void *out, int out_dtype,
                             void *workspace, size_t workspace_bytes, void *stream);

/* The W4A8 gate_up op on activations quantised in token order and read through the row -> token map, as
 * moe355_gmm1_swiglu_quant_gather does for int8 weights: x [T, K] int8, x_scale [T], row_token [rows]. */
int moe355_gmm1_swiglu_quant_w4_gather(const int8_t *x, const float *x_scale, const int32_t *row_token,
                                       const uint8_t *weight_nz4, const float *weight_scale, int64_t group_size,
                                       const float *bias, const int64_t *group_list, int group_list_type,
                                       int64_t rows, int64_t k, int64_t n, int num_experts, float swiglu_limit,
                                       int8_t *out, float *out_scale, void *workspace, size_t workspace_bytes,
                                       void *stream);

/* W4A8 down projection:
 *   out[row, col] = bf16( (sum_g float(acc_g) * scale[e, g, col] + bias[e, col]) * per_token_scale[row] )
 * (the int4 form of torch_npu.npu_grouped_matmul as called from vllm_ascend/ops/fused_moe/moe_mlp.py:552-569). */
int moe355_gmm2_dequant_w4(const int8_t *x, const uint8_t *weight_nz4, const float *scale, int64_t group_size,
                           const float *bias, const float *per_token_scale, const int64_t *group_list,
                           int group_list_type, int64_t rows, int64_t k, int64_t n, int num_experts, void *out,
                           int out_dtype, void *stream);

/* Raw int32 accumulators of the same grouped product (no epilogue):
 * acc [R, N] int32.  The integer stage of both ops above, exposed so a caller
 * can check it exactly (the reference keeps the same intermediate in a global
 * workspace: grouped_matmul_swiglu_quant.h:119,234-265).  The workspace is optional
 * (NULL / 0 is accepted and only costs speed): moe355_gmm_i32_workspace() bytes let the
 * call use the tiled kernels and, for one expert with at most 64 rows, partial sums per
 * slab of K instead of atomics. */
size_t moe355_gmm_i32_workspace(int64_t rows, int64_t n, int64_t k, int num_experts);
int moe355_gmm_i32(const int8_t *x, const int8_t *weight_nz, const int64_t *group_list, int group_list_type,
                   int64_t rows, int64_t k, int64_t n, int num_experts, int32_t *acc, void *workspace,
                   size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * int32 -> dequant -> SwiGLU -> dynamic int8 (the split-path twin of the fused
 * epilogue).  Stands in for torch.ops._C_ascend.npu_dequant_swiglu_quant
 * (schema csrc/torch_binding.cpp:2495-2512) with quant_mode = 1 (dynamic):
 *   f = (float(x) * weight_scale[col]) * activation_scale[row]   (weight scale first:
 *   csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant_dynamic_base.hpp:423-426)
 * x [rows, N] int32; weight_scale [N] fp32; activation_scale [rows] fp32;
 * y [rows, N/2] int8; scale [rows] fp32.  activate_left != 0: SiLU on the left half.
 */
int moe355_dequant_swiglu_quant(const int32_t *x, const float *weight_scale, const float *activation_scale,
                                int64_t rows, int64_t n, int activate_left, float clamp_limit, int8_t *y,
                                float *scale, void *stream);

/* The same op with quant_mode = 0 (static; csrc/moe/dequant_swiglu_quant/op_kernel/
 * dequant_swiglu_quant_static_base.hpp:266-305): after the SwiGLU,
 *   quant_scale_len == n/2:  q = rint(y / quant_scale[col] + quant_offset[col])
 *   quant_scale_len == 1:    q = rint(y * (1 / quant_scale[0]) + quant_offset[0])
 * saturated to int8; quant_offset may be NULL (0).  No scale is written. */
int moe355_dequant_swiglu_quant_static(const int32_t *x, const float *weight_scale, const float *activation_scale,
                                       const float *quant_scale, int64_t quant_scale_len, const float *quant_offset,
                                       int64_t rows, int64_t n, int activate_left, float clamp_limit, int8_t *y,
                                       void *stream);

/* The general form of the same op, as the reference's grouped kernel computes it
 * (csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant.h; Python call site
 * vllm_ascend/ops/fused_moe/moe_mlp.py:340-359 with group_index = the per-expert row counts):
 *   group_index [num_groups] int64 row COUNTS (NULL: one group owning every row); group g owns the next
 *     group_index[g] rows and brings weight_scale[g][n], bias[g][n], quant_scale[g] or [g][n/2]; rows past the
 *     sum get y = 0, scale = 0 (the reference leaves them unwritten)                                (:211-242)
 *   bias_kind 1: int32 bias added to x; 2: fp32 bias added after the scales; 0: none (bias NULL)    (:380-424)
 *   activation_scale may be NULL (no per-row scale)
 *   swiglu_mode 0: lin * silu(act), clamp_limit ignored; 1: lin = clamp(lin, +-clamp_limit) + glu_bias,
 *     act = min(act, clamp_limit) (clamps only when clamp_limit > 0), lin * act / (1 + exp(-glu_alpha * act))  (:627-677)
 *   quant_mode 1: scale = max|v| * (float)(1.0 / 127.0), y = rint(v / scale)                       (:681-738)
 *   quant_mode 0: quant_scale_len == num_groups: y = rint(v * (1 / quant_scale[g]) + quant_offset[g]);
 *     == num_groups * n/2: y = rint(v / quant_scale[g][c] + quant_offset[g][c]); scale is not written (:741-790)
 * A quant_scale in quant_mode 1 (the smooth scale) is MOE355_E_UNSUPPORTED. */
int moe355_dequant_swiglu_quant_grouped(const int32_t *x, const float *weight_scale, const float *activation_scale,
                                        const void *bias, int bias_kind, const int64_t *group_index, int num_groups,
                                        int64_t rows, int64_t n, int activate_left, int swiglu_mode,
                                        float clamp_limit, float glu_alpha, float glu_bias, int quant_mode,
                                        const float *quant_scale, int64_t quant_scale_len, const float *quant_offset,
                                        int8_t *y, float *scale, void *stream);

/* ---------------------------------------------------------------------------
 * Weighted un-permute (finalize routing).
 * Stands in for torch_npu.npu_moe_token_unpermute as called from
 * vllm_ascend/device/device_op.py:950-954 (token_dispatcher.py:451-461; math
 * csrc/mc2/dispatch_ffn_combine/op_kernel/unpermute/moe_token_unpermute.h:241-372):
 *   out[t, :] = bf16( sum_{j=0..k-1, slot order} float(probs[t, j]) * float(permuted[|idx[t*k+j]|, :]) )
 * Slots whose |idx| is not below permuted_rows are skipped, as the reference kernel skips indices >=
 * num_out_tokens (moe_token_unpermute.h:250-275): dropped pairs leave the sum that way.
 * permuted [R, H] bf16 / fp16 (dtype); sorted_indices [T*k] int32; probs [T, k] in the same dtype or NULL
 * (NULL = weight 1); residual [T, H] in the same dtype or NULL is added last in fp32
 * (the shared-expert output; the reference adds it in upstream vLLM).
 */
int moe355_token_unpermute(const void *permuted, int dtype, const int32_t *sorted_indices, const void *probs,
                           int64_t num_tokens, int top_k, int64_t hidden, int64_t permuted_rows,
                           const void *residual, void *out, void *stream);

/* ---------------------------------------------------------------------------
 * Pair order: the expert MLP of a decode batch without a sorted activation.
 * No counterpart of their own in the reference: together with moe355_gate_quant they compute what
 * torch.ops._C_ascend.moe_gating_top_k + torch_npu.npu_moe_init_routing_v2 + grouped_matmul_swiglu_quant +
 * npu_grouped_matmul + npu_moe_token_unpermute compute (vllm_ascend/ops/fused_moe/routed_experts.py:496-609,
 * moe_mlp.py:174-570, token_dispatcher.py:367-461), bit for bit, for at most 1024 (token, slot) pairs
 * (moe355_gmm_pairs_supported() != 0) whose ids all lie in [0, num_experts).  The sort of the pairs by expert,
 * which for such a batch is a hand-off between workgroups through memory in front of the first weight request,
 * disappears: row f = token * top_k + slot of every intermediate tensor belongs to pair f, a workgroup of the
 * weight-streaming GEMM collects the pairs of its expert from topk_ids itself, and the combine reads the k rows of
 * a token where they lie.  A pair whose id is out of range is computed by nobody: its rows are left untouched, and
 * the combine leaves it out of the token's sum and of the counts (a dropped pair, as in the sorted form).
 *   gmm1: x int8 [T, K] and x_scale [T] in token order (moe355_gate_quant) -> out int8 [T*k, N/2], out_scale [T*k]
 *   gmm2: x int8 [T*k, K], per_token_scale [T*k] -> out bf16 / fp16 [T*k, N]
 *   unpermute: out[t] = sum over the slots of token t, in slot order, of probs[t, s] * rows[t*k + s] (+ residual),
 *   the arithmetic of moe355_token_unpermute; expert_tokens [num_experts] int64 receives the number of pairs of
 *   every expert (what moe355_init_routing returns as counts), counted by one more workgroup of the same launch.
 *   num_experts <= 2048. */
int moe355_gmm_pairs_supported(int64_t num_tokens, int top_k, int64_t n, int64_t k);
size_t moe355_gmm1_swiglu_quant_pairs_workspace(int64_t num_tokens, int top_k, int64_t n);
int moe355_gmm1_swiglu_quant_pairs(const int8_t *x, const float *x_scale, const int32_t *topk_ids, int64_t num_tokens,
                                   int top_k, const int8_t *weight_nz, const float *weight_scale, int64_t k,
                                   int64_t n, int num_experts, float swiglu_limit, int8_t *out, float *out_scale,
                                   void *workspace, size_t workspace_bytes, void *stream);
int moe355_gmm2_dequant_pairs(const int8_t *x, const int8_t *weight_nz, const float *scale,
                              const float *per_token_scale, const int32_t *topk_ids, int64_t num_tokens, int top_k,
                              int64_t k, int64_t n, int num_experts, void *out, int out_dtype, void *stream);
/* The same two GEMMs with the re-quantisation inside the second: gmm1 leaves the fp32 SwiGLU values y [T*k, N/2],
 * gmm2 takes them as its activation (K = N/2 of gmm1) and every workgroup quantises the rows of its expert itself
 * (the arithmetic of the re-quantisation of moe355_gmm1_swiglu_quant), so that a decode layer is four launches.
 * moe355_gmm2_requant_pairs_supported() != 0: many units of work, a short K (k < 2048, 32 rows of k + 16 bytes
 * in LDS) and at most three pairs per expert on average -- a small decode batch over many small experts, where a
 * launch costs more than the repeated quantisation. */
int moe355_gmm1_swiglu_pairs(const int8_t *x, const float *x_scale, const int32_t *topk_ids, int64_t num_tokens,
                             int top_k, const int8_t *weight_nz, const float *weight_scale, int64_t k, int64_t n,
                             int num_experts, float swiglu_limit, float *y, void *stream);
int moe355_gmm2_requant_pairs_supported(int64_t num_tokens, int top_k, int64_t n, int64_t k, int num_experts);
int moe355_gmm2_requant_dequant_pairs(const float *y, const int8_t *weight_nz, const float *scale,
                                      const int32_t *topk_ids, int64_t num_tokens, int top_k, int64_t k, int64_t n,
                                      int num_experts, void *out, int out_dtype, void *stream);
int moe355_token_unpermute_pairs(const void *rows, int dtype, const void *probs, const int32_t *topk_ids,
                                 int64_t num_tokens, int top_k, int64_t hidden, int num_experts, const void *residual,
                                 void *out, int64_t *expert_tokens, void *stream);

/* ---------------------------------------------------------------------------
 * Measurement hook (no counterpart in the reference; for benchmarks).  The one piece of per-thread host
 * state in the library: the armed pair of events is kept in thread-local storage until the next GEMM launch
 * of the same thread takes it.
 * The next grouped-GEMM kernel launched from the calling thread by
 * moe355_gmm1_swiglu_quant / moe355_gmm2_dequant / moe355_gmm_i32 is bracketed
 * by the two hipEvent_t handles (recorded immediately before and after that
 * one kernel, not the small helper kernels around it).  One-shot: the pair is
 * consumed by that launch.  Pass two NULLs to cancel.
 */
int moe355_profile_next_gemm(void *start_event, void *stop_event);

/* Which kernel family the int8 grouped GEMMs above launch for a shape, given a workspace of the size their
 * moe355_*_workspace() asks for: "gmm_stream_kernel" (few rows per expert), "gmm_tiled_kernel" (128-row
 * LDS-tiled), "gmm_wide_kernel" (weight-streaming tiles of up to 256 rows) or "gmm_dense_kernel" (one expert
 * with thousands of rows: 256 x 256 tiles, no tile map); "" for arguments no GEMM accepts.
 * epilogue: 0 raw int32 (moe355_gmm_i32), 1 SwiGLU (moe355_gmm1_swiglu_quant), 2 dequant (moe355_gmm2_dequant).
 * A pure function of its arguments, for benchmarks and profiles (no counterpart in the reference). */
const char *moe355_gmm_kernel_name(int epilogue, int64_t rows, int64_t k, int64_t n, int num_experts);

#ifdef __cplusplus
}
#endif
#endif /* MOE355_H */
