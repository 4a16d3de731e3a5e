/*
 * moe_oracle.c -- CPU restatement of the W8A8-dynamic fused-MoE layer.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU kernels are
 * compared against.  Nothing in the shipped package links, imports or calls
 * it; only the tests, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * Every function cites the reference file (paths under the vllm-ascend tree)
 * whose arithmetic it restates.  Where the reference leaves a choice to a
 * closed third-party binary (torch_npu / CANN), the rule fixed here is marked
 * [fixed by build].
 *
 * Arithmetic contract: IEEE-754 binary32, round-to-nearest-even, no
 * contraction of a multiply and an add into a fused operation (compile with
 * -ffp-contract=off).  Fused multiply-adds exist only where fmaf() is written
 * out: the range reduction and the polynomial of the shared exp() (orc_expf)
 * and the dot products of the router gate (orc_router_gate); a GPU kernel that
 * executes the same sequence with v_fma_f32 in the same places gives the same
 * bits.
 *
 * Parity pins (what checks each function against something other than itself;
 * the tests live in tests/test_oracle_*.py):
 *   orc_expf            : libm expf within 2 ulp on a dense grid of [-87, 88.7] + the clamps
 *   orc_gating_top_k    : numpy rendering of the reference golden function
 *                         (tests/e2e/nightly/single_node/ops/singlecard_ops/
 *                         test_npu_moe_gating_top_k.py:33-112) over its grid,
 *                         brute-force enumeration on tiny inputs, closed forms
 *   orc_init_routing    : known-answer vector tests/ut/lora/test_lora.py:151-165,
 *                         numpy stable argsort, bincount; dropped (out-of-range) ids against a
 *                         filtered numpy sort
 *   orc_dynamic_quant   : closed forms (identity rows, zero rows, .5 ties)
 *                         rounding rule itself: PARITY UNPINNED (torch_npu binary)
 *   orc_gmm_i32         : numpy int64 matmul (exact)
 *   orc_silu            : float64 g / (1 + exp(-g)) within 3 units in the last place on a dense grid,
 *                         the closed forms silu(g) = g for g >= 17.4, silu(0) = 0, silu(-0) = -0 and the
 *                         values orc_swiglu_quant returns for the same gates (one expression, two places)
 *   orc_swiglu_quant    : numpy rendering of the reference golden
 *                         (test_gmm_swiglu_quant_weight_nz_tensor_list.py:14-99), +-1 LSB
 *   orc_gmm2_dequant    : numpy float64 product, bf16 rounding closed forms
 *                         multiplication order: PARITY UNPINNED (torch_npu binary)
 *   orc_unpermute       : dense torch_moe restatement (test_fused_moe.py:85-97); the residual
 *                         add: exact small-integer cases, a case that tells "added last in fp32"
 *                         from "added after rounding" and from "added first"; skipped rows
 *                         accumulation order: PARITY UNPINNED (torch_npu binary)
 *   orc_dequant_swiglu_quant : numpy rendering of test_dequant_swiglu_quant.py:16-45, both
 *                         values of activate_left (the golden's own branch, and the identity
 *                         "swap the halves of x and of the weight scale")
 *   orc_dequant_swiglu_quant_static : the dynamic mode's SwiGLU values (orc_swiglu_quant's y) pushed through
 *                         numpy's y / scale + offset and rint, per-channel and per-tensor, with and without offset
 *   orc_dequant_swiglu_quant_grouped : with one group, no bias and swiglu_mode 0 the SwiGLU values of
 *                         orc_dequant_swiglu_quant; with groups, the same function called per row range with that
 *                         group's scales (numpy slicing); int32 bias = the op on x + bias; float64 closed form of
 *                         the swiglu_mode 1 expression (clamps, alpha, bias) within fp32 rounding; the quantiser's
 *                         own arithmetic (max * (1/127), v / scale) against numpy float32
 *   orc_erff, orc_tanhf : math.erf within 5e-7, math.tanh within 3e-7 absolute on a dense grid, odd symmetry, the limits
 *   orc_act_mul_quant   : float64 formulas of the four activations within 16-bit rounding, clamp closed forms,
 *                         the quantiser of orc_dynamic_quant on the rounded values; which intermediate roundings
 *                         the reference's closed kernels apply: PARITY UNPINNED
 *   shared expert (oracle.py: shared_expert_forward, composed of the functions above in the order of
 *                         vllm_ascend/ops/fused_moe/shared_experts.py:254-301): dense float64 MLP on the
 *                         dequantised weights within the quantisation noise, exact agreement with the
 *                         grouped path run with one expert (which differs only in the order of the two
 *                         scale multiplications) on power-of-two scales
 *   orc_router_gate     : float64 dot products (tolerance), exact integer cases, cases that tell the
 *                         chunked fma order from a plain ascending sum, from multiply-then-add and from
 *                         other chunk lengths; the order itself: PARITY UNPINNED (F.linear's BLAS)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ helpers */

static inline float bits_to_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet). */
static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7f800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> fp16, round to nearest even. */
static inline uint16_t f32_to_f16(float f)
{
    uint32_t u = f32_to_bits(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 rounds up too, handled below) */
    if (a < 0x33000000u) return (uint16_t)sign;              /* < 2^-25 -> 0 */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t half = 1u << (shift - 1);
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t q = m >> shift;
    if (rem > half || (rem == half && (q & 1u))) q++;
    uint32_t out;
    if (e < -14) {
        out = q; /* subnormal (q may carry into exponent 1, which is correct) */
    } else {
        out = ((uint32_t)(e + 15) << 10) + (q - 0x400u);
    }
    if (out >= 0x7c00u) out = 0x7c00u;
    return (uint16_t)(sign | out);
}

/*
 * exp(x) in binary32 as one fixed sequence of operations [fixed by build].
 * The argument is first clamped to [-87, 88.72283] (so the result is always a normal
 * number or +inf; a NaN argument is treated as -87), then Cephes-style: n = rint(x*log2e),
 * Cody-Waite reduction with a two-part ln2, degree-5 polynomial, exact scaling by 2^n
 * (ldexp).  Every multiply-add of the reduction and of the polynomial is ONE fused operation
 * (fmaf: a single rounding), written out explicitly; the GPU kernels run the identical sequence
 * (v_fma_f32), so both sides agree bit for bit.
 */
ORC_API float orc_expf(float x)
{
    x = fminf(fmaxf(x, -87.0f), 88.72283f);
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    float y = fmaf(p, r2, r);
    y = y + 1.0f;
    return ldexpf(y, (int)n);
}

/* Which 16-bit float the layer's hidden states use: 0 = bf16 (default), 1 = fp16.  The functions that read or
 * write hidden states (quantiser, gather, down projection, combine, router gate) go through h2f / f2h; the
 * reference supports both (the model dtype).  Set from the tests through orc_set_half_kind. */
static int g_half_is_f16 = 0;
ORC_API void orc_set_half_kind(int is_f16) { g_half_is_f16 = is_f16 != 0; }
ORC_API int orc_get_half_kind(void) { return g_half_is_f16; }
static inline float h2f(uint16_t h) { return g_half_is_f16 ? f16_to_f32(h) : bf16_to_f32(h); }
static inline uint16_t f2h(float f) { return g_half_is_f16 ? f32_to_f16(f) : f32_to_bf16(f); }

/*
 * Sum of n floats in the one order every implementation of this layer uses
 * [fixed by build]: 64 strided partial sums (partial[l] adds v[l], v[l+64], ...
 * in ascending index, starting from +0), then a butterfly: for off = 32,16,..,1
 * every partial becomes partial[l] + partial[l ^ off].  All 64 end up equal.
 */
static float wave_tree_sum(const float *v, int n)
{
    float part[64], nxt[64];
    for (int l = 0; l < 64; ++l) {
        float s = 0.0f;
        for (int i = l; i < n; i += 64) s = s + v[i];
        part[l] = s;
    }
    for (int off = 32; off >= 1; off >>= 1) {
        for (int l = 0; l < 64; ++l) nxt[l] = part[l] + part[l ^ off];
        memcpy(part, nxt, sizeof(part));
    }
    return part[0];
}

ORC_API float orc_wave_tree_sum(const float *v, int n) { return wave_tree_sum(v, n); }

/* ------------------------------------------------------------------ routing */

/* "a ranks before b": larger value first, ties to the lower index. */
static inline int ranks_before(float va, int ia, float vb, int ib)
{
    if (va > vb) return 1;
    if (va < vb) return 0;
    return ia < ib;
}

/*
 * Group-limited top-k gating.
 * Restates csrc/moe/moe_gating_top_k/op_kernel/moe_gating_top_k_generalized.h:153-226
 * (normalisation: softmax = exp(x-max) * (1/sum), sigmoid; bias added for
 * selection only), :264-340 (group score = max or sum of the two largest, keep
 * k_group groups, the rest masked to -inf), :518-557 (gather the unbiased
 * scores, divide by (sum + eps) when sigmoid or renorm, multiply by the routed
 * scaling factor) and the golden function
 * tests/e2e/nightly/single_node/ops/singlecard_ops/test_npu_moe_gating_top_k.py:33-112
 * (stable descending order: ties go to the lower index).
 *
 * x    [T,E] fp32 (already widened from the caller's dtype)
 * bias [E] fp32 or NULL
 * y    [T,k] fp32 (the caller narrows it to the logits dtype, RNE)
 * idx  [T,k] int32
 * norm [T,E] fp32 normalised scores, or NULL
 */
ORC_API int orc_gating_top_k(const float *x, const float *bias, int64_t T, int E, int k, int k_group, int group_count,
                             int group_select_mode, int renorm, int norm_type, float routed_scaling_factor, float eps,
                             float *y, int32_t *idx, float *norm)
{
    if (E <= 0 || k <= 0 || k > E || group_count <= 0 || E % group_count != 0) return -1;
    if (k_group <= 0 || k_group > group_count) return -1;
    if (norm_type != 0 && norm_type != 1) return -1;
    const int gs = E / group_count;
    float *p = (float *)malloc(sizeof(float) * (size_t)E);
    float *sel = (float *)malloc(sizeof(float) * (size_t)E);
    float *gscore = (float *)malloc(sizeof(float) * (size_t)group_count);
    unsigned char *gkeep = (unsigned char *)malloc((size_t)group_count);
    unsigned char *taken = (unsigned char *)malloc((size_t)E);
    for (int64_t t = 0; t < T; ++t) {
        const float *row = x + t * E;
        if (norm_type == 0) {
            float m = row[0];
            for (int e = 1; e < E; ++e) m = row[e] > m ? row[e] : m;
            for (int e = 0; e < E; ++e) p[e] = orc_expf(row[e] - m);
            float s = wave_tree_sum(p, E);
            float inv = 1.0f / s;
            for (int e = 0; e < E; ++e) p[e] = p[e] * inv;
        } else {
            for (int e = 0; e < E; ++e) p[e] = 1.0f / (1.0f + orc_expf(-row[e]));
        }
        if (norm) memcpy(norm + t * E, p, sizeof(float) * (size_t)E);
        for (int e = 0; e < E; ++e) sel[e] = bias ? p[e] + bias[e] : p[e];

        if (group_count > 1) {
            for (int g = 0; g < group_count; ++g) {
                const float *s = sel + g * gs;
                int i1 = 0;
                for (int j = 1; j < gs; ++j)
                    if (ranks_before(s[j], j, s[i1], i1)) i1 = j;
                if (group_select_mode == 0 || gs < 2) {
                    gscore[g] = s[i1];
                } else {
                    int i2 = (i1 == 0) ? 1 : 0;
                    for (int j = 0; j < gs; ++j)
                        if (j != i1 && ranks_before(s[j], j, s[i2], i2)) i2 = j;
                    gscore[g] = s[i1] + s[i2];
                }
            }
            memset(gkeep, 0, (size_t)group_count);
            for (int c = 0; c < k_group; ++c) {
                int best = -1;
                for (int g = 0; g < group_count; ++g) {
                    if (gkeep[g]) continue;
                    if (best < 0 || ranks_before(gscore[g], g, gscore[best], best)) best = g;
                }
                gkeep[best] = 1;
            }
            for (int g = 0; g < group_count; ++g)
                if (!gkeep[g])
                    for (int j = 0; j < gs; ++j) sel[g * gs + j] = -INFINITY;
        }

        memset(taken, 0, (size_t)E);
        float wsum = 0.0f;
        for (int c = 0; c < k; ++c) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                if (taken[e]) continue;
                if (best < 0 || ranks_before(sel[e], e, sel[best], best)) best = e;
            }
            taken[best] = 1;
            idx[t * k + c] = best;
            y[t * k + c] = p[best];
            wsum = wsum + p[best];
        }
        if (norm_type == 1 || renorm == 1) {
            float d = wsum + eps;
            for (int c = 0; c < k; ++c) y[t * k + c] = y[t * k + c] / d;
        }
        for (int c = 0; c < k; ++c) y[t * k + c] = y[t * k + c] * routed_scaling_factor;
    }
    free(p);
    free(sel);
    free(gscore);
    free(gkeep);
    free(taken);
    return 0;
}

/* ------------------------------------------------------------------ quantiser */

/*
 * Per-row dynamic int8 quantisation [fixed by build; the rounding inside
 * torch_npu.npu_dynamic_quant / npu_moe_init_routing_v2(quant_mode=1) is not
 * visible in the reference -- PARITY UNPINNED for the rounding rule].
 * Follows the shape of
 * csrc/mc2/dispatch_ffn_combine/op_kernel/moe_init_routing_quant_v2/moe_v2_gather_dynamic_quant.h:116-155
 * (scale = absmax/127, q = x/scale rounded) with one rounding, to nearest even:
 *   a = max|v| ; s = a/127.0f ; q = clamp(rint(v/s), -128, 127) ; a == 0 -> q = 0, s = 0.
 */
static void quant_row_f32(const float *v, int64_t n, int8_t *q, float *scale)
{
    float a = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        float b = fabsf(v[i]);
        a = b > a ? b : a;
    }
    if (a == 0.0f) {
        memset(q, 0, (size_t)n);
        *scale = 0.0f;
        return;
    }
    float s = a / 127.0f;
    for (int64_t i = 0; i < n; ++i) {
        float r = rintf(v[i] / s);
        r = r > 127.0f ? 127.0f : r;
        r = r < -128.0f ? -128.0f : r;
        q[i] = (int8_t)r;
    }
    *scale = s;
}

ORC_API int orc_dynamic_quant_bf16(const uint16_t *x, int64_t rows, int64_t cols, int8_t *q, float *scale)
{
#pragma omp parallel
    {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)cols);
#pragma omp for
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t c = 0; c < cols; ++c) tmp[c] = h2f(x[r * cols + c]);
            quant_row_f32(tmp, cols, q + r * cols, scale + r);
        }
        free(tmp);
    }
    return 0;
}

/*
 * Expert histogram + stable sort of the flattened [T*k] expert ids + gather
 * with fused per-row quantisation.
 * Restates the contract of torch_npu.npu_moe_init_routing_v2 as the reference
 * uses it (vllm_ascend/ops/fused_moe/token_dispatcher.py:367-449, quant_mode=1,
 * expert_tokens_num_type=1 "count"), the permutation contract documented at
 * vllm_ascend/lora/fused_moe.py:190-204 and the in-repo AscendC rendering
 * csrc/mc2/dispatch_ffn_combine/op_kernel/moe_init_routing_quant_v2/moe_v2_sort_one_core.h:42-99,
 * moe_v2_src_to_dst_op.h:68-104:
 *   dst[f] = position of flat pair f = t*k+j after a stable sort by expert id.
 *
 * ids [R] int32 (R = T*k), dst [R] int32, cnt [E] int64,
 * x [T,H] bf16, xs [R,H] int8 (or NULL to skip the gather), sx [R] fp32.
 */
ORC_API int orc_init_routing(const int32_t *ids, int64_t T, int k, int E, const uint16_t *x, int64_t H, int32_t *dst,
                             int64_t *cnt, int8_t *xs, float *sx)
{
    const int64_t R = T * k;
    int64_t *off = (int64_t *)calloc((size_t)E + 1, sizeof(int64_t));
    for (int e = 0; e < E; ++e) cnt[e] = 0;
    /* a pair whose expert id lies outside [0, E) is dropped: it is not counted, its row is not written and its
     * destination is R, one past the last row (an index the combine skips) */
    for (int64_t f = 0; f < R; ++f)
        if (ids[f] >= 0 && ids[f] < E) cnt[ids[f]]++;
    for (int e = 0; e < E; ++e) off[e + 1] = off[e] + cnt[e];
    for (int64_t f = 0; f < R; ++f) dst[f] = (ids[f] >= 0 && ids[f] < E) ? (int32_t)(off[ids[f]]++) : (int32_t)R;
    free(off);
    if (xs && x) {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)H);
        int8_t *qrow = (int8_t *)malloc((size_t)H);
        for (int64_t t = 0; t < T; ++t) {
            float s;
            for (int64_t c = 0; c < H; ++c) tmp[c] = h2f(x[t * H + c]);
            quant_row_f32(tmp, H, qrow, &s);
            for (int j = 0; j < k; ++j) {
                int64_t d = dst[t * k + j];
                if (d >= R) continue;
                memcpy(xs + d * H, qrow, (size_t)H);
                sx[d] = s;
            }
        }
        free(tmp);
        free(qrow);
    }
    return 0;
}

/* Same permutation without quantisation (quant_mode = -1): rows copied as bf16. */
ORC_API int orc_permute_rows_bf16(const int32_t *dst, int64_t T, int k, const uint16_t *x, int64_t H, uint16_t *xp)
{
    for (int64_t t = 0; t < T; ++t)
        for (int j = 0; j < k; ++j)
            if ((int64_t)dst[t * k + j] < T * k) memcpy(xp + (int64_t)dst[t * k + j] * H, x + t * H, (size_t)H * 2);
    return 0;
}

/* ------------------------------------------------------------------ grouped GEMM */

/* expert of row r given the cumulative group list (first e with r < cum[e]); E if none. */
static inline int expert_of_row(const int64_t *cum, int E, int64_t r)
{
    int lo = 0, hi = E;
    while (lo < hi) {
        int mid = (lo + hi) / 2;
        if (r < cum[mid])
            hi = mid;
        else
            lo = mid + 1;
    }
    return lo;
}

/*
 * Exact int8 x int8 -> int32 grouped matmul:  acc[r,n] = sum_k x[r,k] * w[e(r),n,k].
 * Restates the integer stage of
 * csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:234-265
 * and of torch_npu.npu_grouped_matmul as called from vllm_ascend/device/device_op.py:254-291.
 * w is [E,N,K] (checkpoint order, K contiguous); cum is the cumulative group list [E].
 * Rows >= cum[E-1] are left untouched.
 */
ORC_API int orc_gmm_i32(const int8_t *x, const int8_t *w, const int64_t *cum, int64_t R, int64_t K, int64_t N, int E,
                        int32_t *acc)
{
    int64_t rows = cum[E - 1] < R ? cum[E - 1] : R;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t r = 0; r < rows; ++r) {
        int e = expert_of_row(cum, E, r);
        const int8_t *xr = x + r * K;
        const int8_t *we = w + (int64_t)e * N * K;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t *wn = we + n * K;
            int32_t s = 0;
            for (int64_t kk = 0; kk < K; ++kk) s += (int32_t)xr[kk] * (int32_t)wn[kk];
            acc[r * N + n] = s;
        }
    }
    return 0;
}

/*
 * W4A8 integer stage with per-group fp32 scales (group size gsz along K):
 *   f[r,n] = sum_g float( sum_{k in g} x[r,k]*w[e,n,k] ) * sg[e,g,n]     (g ascending, fp32)
 * Restates custom_mm's per-group branch of
 * tests/e2e/nightly/single_node/ops/singlecard_ops/test_grouped_matmul_swiglu_quant.py:22-55
 * in fp32 (the Ascend kernel accumulates in fp16 because of its int4 cube; the
 * intended mathematics is the fp32 sum, csrc/gmm/grouped_matmul_swiglu_quant/README.md).
 * w holds int4 values (-8..7) already unpacked to one int8 each, [E,N,K].
 * sg is [E,K/gsz,N].
 */
ORC_API int orc_gmm_w4_grouped(const int8_t *x, const int8_t *w, const float *sg, const int64_t *cum, int64_t R,
                               int64_t K, int64_t N, int E, int64_t gsz, float *f)
{
    if (K % gsz != 0) return -1;
    const int64_t G = K / gsz;
    int64_t rows = cum[E - 1] < R ? cum[E - 1] : R;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t r = 0; r < rows; ++r) {
        int e = expert_of_row(cum, E, r);
        const int8_t *xr = x + r * K;
        for (int64_t n = 0; n < N; ++n) {
            const int8_t *wn = w + ((int64_t)e * N + n) * K;
            float tot = 0.0f;
            for (int64_t g = 0; g < G; ++g) {
                int32_t s = 0;
                for (int64_t kk = g * gsz; kk < (g + 1) * gsz; ++kk) s += (int32_t)xr[kk] * (int32_t)wn[kk];
                tot = tot + (float)s * sg[((int64_t)e * G + g) * N + n];
            }
            f[r * N + n] = tot;
        }
    }
    return 0;
}

/*
 * Dequant of the gate_up accumulator: token scale first, then channel scale.
 * Restates csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:387-399
 * (x_scale) and :448-459 (weight_scale).   f = (float(acc) * sx[r]) * sw[e,n].
 */
ORC_API int orc_dequant_acc(const int32_t *acc, const float *sx, const float *sw, const int64_t *cum, int64_t R,
                            int64_t N, int E, float *f)
{
    int64_t rows = cum[E - 1] < R ? cum[E - 1] : R;
#pragma omp parallel for
    for (int64_t r = 0; r < rows; ++r) {
        int e = expert_of_row(cum, E, r);
        for (int64_t n = 0; n < N; ++n) {
            float v = (float)acc[r * N + n];
            v = v * sx[r];
            v = v * sw[(int64_t)e * N + n];
            f[r * N + n] = v;
        }
    }
    return 0;
}

/* multiply every element of row r by sx[r] (the W4A8 path applies the token scale last). */
ORC_API int orc_scale_rows(float *f, const float *sx, int64_t rows, int64_t N)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t n = 0; n < N; ++n) f[r * N + n] = f[r * N + n] * sx[r];
    return 0;
}

/*
 * SwiGLU + per-row dynamic int8 re-quantisation of dequantised gate_up values.
 * Restates csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:461-520
 * and csrc/gmm/grouped_matmul_swiglu_quant/README.md:63-67: the first N/2
 * columns are the gate, the second N/2 the up projection,
 *   y = (g / (1 + exp(-g))) * u ;  s = max|y| / 127 ;  q = rint(y * (1/s)).
 * swiglu_limit > 0 clamps g to (-inf, L] and u to [-L, L] first.
 * The Ascend fp32->fp16->int8 detour (grouped_matmul_swiglu_quant_utils.h:308-325)
 * is not reproduced; one RNE rounding, saturating [fixed by build].
 * yout (optional) receives the fp32 SwiGLU values [rows, N/2].
 */
ORC_API int orc_swiglu_quant(const float *f, int64_t rows, int64_t N, float swiglu_limit, int8_t *q, float *qs,
                             float *yout)
{
    const int64_t I = N / 2;
#pragma omp parallel
    {
        float *y = (float *)malloc(sizeof(float) * (size_t)I);
#pragma omp for
        for (int64_t r = 0; r < rows; ++r) {
            const float *fr = f + r * N;
            float a = 0.0f;
            for (int64_t i = 0; i < I; ++i) {
                float g = fr[i], u = fr[I + i];
                if (swiglu_limit > 0.0f) {
                    g = g > swiglu_limit ? swiglu_limit : g;
                    u = u > swiglu_limit ? swiglu_limit : u;
                    u = u < -swiglu_limit ? -swiglu_limit : u;
                }
                float sg = g / (1.0f + orc_expf(-g));
                float v = sg * u;
                y[i] = v;
                float b = fabsf(v);
                a = b > a ? b : a;
            }
            if (yout) memcpy(yout + r * I, y, sizeof(float) * (size_t)I);
            if (a == 0.0f) {
                memset(q + r * I, 0, (size_t)I);
                qs[r] = 0.0f;
                continue;
            }
            float s = a / 127.0f;
            float inv = 1.0f / s;
            for (int64_t i = 0; i < I; ++i) {
                float t = rintf(y[i] * inv);
                t = t > 127.0f ? 127.0f : t;
                t = t < -128.0f ? -128.0f : t;
                q[r * I + i] = (int8_t)t;
            }
            qs[r] = s;
        }
        free(y);
    }
    return 0;
}

/*
 * The gate function of the SwiGLU by itself, element by element: out[i] = g[i] / (1 + exp(-g[i])) with the
 * IEEE division of C (README formula csrc/gmm/grouped_matmul_swiglu_quant/README.md:63-67, kernel
 * csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant.h:461-485).  The same expression
 * as inside orc_swiglu_quant; exported so that the GPU's instruction sequence for it can be compared on
 * arbitrary bit patterns.
 */
ORC_API int orc_silu(const float *g, int64_t n, float *out)
{
#pragma omp parallel for
    for (int64_t i = 0; i < n; ++i) out[i] = g[i] / (1.0f + orc_expf(-g[i]));
    return 0;
}

/*
 * Down-projection dequant to bf16 [multiplication order fixed by build: the
 * order inside torch_npu.npu_grouped_matmul is not visible -- PARITY UNPINNED]:
 *   o[r,h] = bf16( (float(acc) * s1[r]) * s2[e,h] ).
 * Call site: vllm_ascend/ops/fused_moe/moe_mlp.py:552-569, vllm_ascend/device/device_op.py:254-291.
 */
ORC_API int orc_gmm2_dequant(const int32_t *acc, const float *s1, const float *s2, const int64_t *cum, int64_t R,
                             int64_t N, int E, uint16_t *o)
{
    int64_t rows = cum[E - 1] < R ? cum[E - 1] : R;
#pragma omp parallel for
    for (int64_t r = 0; r < rows; ++r) {
        int e = expert_of_row(cum, E, r);
        for (int64_t n = 0; n < N; ++n) {
            float v = (float)acc[r * N + n];
            v = v * s1[r];
            v = v * s2[(int64_t)e * N + n];
            o[r * N + n] = f2h(v);
        }
    }
    return 0;
}

/*
 * Weighted un-permute / finalize:
 *   out[t,:] = bf16( sum_{j=0..k-1 in slot order} float(w[t,j]) * float(o[dst[t*k+j],:]) ), fp32 accumulate.
 * Restates csrc/mc2/dispatch_ffn_combine/op_kernel/unpermute/moe_token_unpermute.h:241-372;
 * call site vllm_ascend/ops/fused_moe/token_dispatcher.py:451-461.  [accumulation
 * order inside torch_npu.npu_moe_token_unpermute is not visible -- PARITY UNPINNED]
 * add (optional, [T,H] bf16) is added last in fp32 (shared-expert output).
 * o has `rows` rows; an index whose magnitude is not below `rows` is skipped, as the reference kernel skips
 * indices >= num_out_tokens (moe_token_unpermute.h:250-275): that is how dropped pairs leave the sum.
 */
ORC_API int orc_unpermute(const uint16_t *o, int64_t rows, const int32_t *dst, const uint16_t *w, int64_t T, int k,
                          int64_t H, const uint16_t *add, uint16_t *out)
{
#pragma omp parallel for
    for (int64_t t = 0; t < T; ++t) {
        for (int64_t h = 0; h < H; ++h) {
            float acc = 0.0f;
            for (int j = 0; j < k; ++j) {
                int64_t d = dst[t * k + j];
                d = d < 0 ? -d : d;
                if (d >= rows) continue;
                float p = h2f(w[t * k + j]) * h2f(o[d * H + h]);
                acc = acc + p;
            }
            if (add) acc = acc + h2f(add[t * H + h]);
            out[t * H + h] = f2h(acc);
        }
    }
    return 0;
}

/*
 * Split-path twin of the fused epilogue: int32 -> dequant -> SwiGLU -> dynamic int8.
 * Restates csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant_dynamic_base.hpp:423-426
 * (weight scale first, then activation scale -- the opposite order from the
 * fused grouped op) and the golden
 * tests/e2e/nightly/single_node/ops/singlecard_ops/test_dequant_swiglu_quant.py:16-45.
 * activate_left: the SiLU is applied to the left half.  quant_mode 1 = dynamic.
 */
ORC_API int orc_dequant_swiglu_quant(const int32_t *x, const float *w_scale, const float *a_scale, int64_t rows,
                                     int64_t N, int activate_left, float clamp_limit, int8_t *q, float *qs)
{
    float *f = (float *)malloc(sizeof(float) * (size_t)rows * (size_t)N);
    const int64_t I = N / 2;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t n = 0; n < N; ++n) {
            float v = (float)x[r * N + n];
            v = v * w_scale[n];
            v = v * a_scale[r];
            /* orc_swiglu_quant applies SiLU to the first half */
            int64_t c = activate_left ? n : (n < I ? n + I : n - I);
            f[r * N + c] = v;
        }
    int rc = orc_swiglu_quant(f, rows, N, clamp_limit, q, qs, NULL);
    free(f);
    return rc;
}

/*
 * The static quantisation mode of the same op (quant_mode 0; the mode string "static" of
 * csrc/moe/dequant_swiglu_quant/op_host/dequant_swiglu_quant_def.cpp:95).  Restates
 * csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant_static_base.hpp:266-305: after the SwiGLU,
 *   one scale per output channel (n_quant == N/2):  v = y / quant_scale[c] + quant_offset[c]
 *   one scale for the tensor     (n_quant == 1):    v = y * (1 / quant_scale[0]) + quant_offset[0]
 *   q = rint(v), saturated to int8 [one rounding, fixed by build: the kernel goes fp32 -> int16 -> fp16 -> int8].
 * quant_offset may be NULL (0).  No scale is returned.
 */
ORC_API int orc_dequant_swiglu_quant_static(const int32_t *x, const float *w_scale, const float *a_scale,
                                            const float *quant_scale, int64_t n_quant, const float *quant_offset,
                                            int64_t rows, int64_t N, int activate_left, float clamp_limit, int8_t *q)
{
    const int64_t I = N / 2;
    const float inv0 = 1.0f / quant_scale[0];
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t i = 0; i < I; ++i) {
            const int64_t gi = activate_left ? i : i + I, ui = activate_left ? i + I : i;
            float g = ((float)x[r * N + gi] * w_scale[gi]) * a_scale[r];
            float u = ((float)x[r * N + ui] * w_scale[ui]) * a_scale[r];
            if (clamp_limit > 0.0f) {
                g = g > clamp_limit ? clamp_limit : g;
                u = u > clamp_limit ? clamp_limit : u;
                u = u < -clamp_limit ? -clamp_limit : u;
            }
            float y = (g / (1.0f + orc_expf(-g))) * u;
            float v;
            if (n_quant == 1) v = y * inv0 + (quant_offset ? quant_offset[0] : 0.0f);
            else v = y / quant_scale[i] + (quant_offset ? quant_offset[i] : 0.0f);
            float t = rintf(v);
            t = t > 127.0f ? 127.0f : t;
            t = t < -128.0f ? -128.0f : t;
            q[r * I + i] = (int8_t)t;
        }
    return 0;
}

/*
 * The general form of npu_dequant_swiglu_quant: rows in groups with a weight scale (bias, quant scale) per group,
 * int32 or float bias, the clamped / scaled SwiGLU of swiglu_mode 1.  Restates the kernel class every grouped
 * call runs, csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant.h (dispatch:
 * dequant_swiglu_quant.cpp:77-171):
 *   groups      group_index holds row COUNTS (negative = 0); group g owns the next count rows; rows past the sum
 *               are not processed (here: y = 0, scale = 0)                                         (:211-242)
 *   dequant     int32 bias is added to x first; f = float(x) * weight_scale[g][c], then * activation_scale[row]
 *               when there is one; a float bias is added after both                               (:380-424)
 *   swiglu 0    lin * (act / (1 + exp(-act))), no clamp                                             (:432-470)
 *   swiglu 1    lin = clamp(lin, -L, L) + glu_bias;  act = min(act, L)  (both only when L > 0);
 *               lin * (act / (1 + exp(act * -glu_alpha)))                                           (:627-677)
 *   dynamic     scale = max|v| * (float)(1.0 / 127.0);  q = rint(v / scale)                         (:681-738)
 *   static      one scale per group: q = rint(v * (1 / quant_scale[g]) + quant_offset[g]);
 *               per channel: q = rint(v / quant_scale[g][c] + quant_offset[g][c])                   (:277-324, :741-790)
 * "act" is the left half when activate_left, else the right one.  bias_kind: 0 none, 1 int32, 2 float.
 * An all-zero row has scale 0 and q = 0 (fixed by build: the kernel divides by zero there).
 */
ORC_API int orc_dequant_swiglu_quant_grouped(const int32_t *x, const float *w_scale, const float *a_scale,
                                             const void *bias, int bias_kind, const int64_t *group_index,
                                             int64_t num_groups, int64_t rows, int64_t N, int activate_left,
                                             int swiglu_mode, float clamp_limit, float glu_alpha, float glu_bias,
                                             int quant_mode, const float *quant_scale, int quant_per_channel,
                                             const float *quant_offset, int8_t *q, float *qs)
{
    const int64_t I = N / 2;
    const float factor = (float)(1.0 / 127.0);
    float *v = (float *)malloc(sizeof(float) * (size_t)(I > 0 ? I : 1));
    int64_t g = 0, left = (group_index && num_groups > 0) ? (group_index[0] < 0 ? 0 : group_index[0]) : rows;
    for (int64_t r = 0; r < rows; ++r) {
        if (group_index) {
            while (g < num_groups && left == 0) {
                ++g;
                if (g < num_groups) left = group_index[g] < 0 ? 0 : group_index[g];
            }
            if (g >= num_groups) { /* past the last group */
                memset(q + r * I, 0, (size_t)I);
                if (qs) qs[r] = 0.0f;
                continue;
            }
            --left;
        }
        const float *ws = w_scale + g * N;
        float amax = 0.0f;
        for (int64_t i = 0; i < I; ++i) {
            const int64_t ai = activate_left ? i : i + I, li = activate_left ? i + I : i;
            int32_t xa = x[r * N + ai], xl = x[r * N + li];
            if (bias_kind == 1) {
                xa = (int32_t)((uint32_t)xa + (uint32_t)((const int32_t *)bias)[g * N + ai]);
                xl = (int32_t)((uint32_t)xl + (uint32_t)((const int32_t *)bias)[g * N + li]);
            }
            float act = (float)xa * ws[ai], lin = (float)xl * ws[li];
            if (a_scale) {
                act = act * a_scale[r];
                lin = lin * a_scale[r];
            }
            if (bias_kind == 2) {
                act = act + ((const float *)bias)[g * N + ai];
                lin = lin + ((const float *)bias)[g * N + li];
            }
            float e;
            if (swiglu_mode == 1) {
                if (clamp_limit > 0.0f) {
                    lin = lin > clamp_limit ? clamp_limit : lin;
                    lin = lin < -clamp_limit ? -clamp_limit : lin;
                }
                lin = lin + glu_bias;
                if (clamp_limit > 0.0f) act = act > clamp_limit ? clamp_limit : act;
                e = orc_expf(act * -glu_alpha);
            } else {
                e = orc_expf(act * -1.0f);
            }
            v[i] = lin * (act / (1.0f + e));
            const float a = fabsf(v[i]);
            amax = a > amax ? a : amax;
        }
        if (quant_mode == 1) {
            const float scale = amax * factor;
            qs[r] = amax == 0.0f ? 0.0f : scale;
            for (int64_t i = 0; i < I; ++i) {
                float t = amax == 0.0f ? 0.0f : rintf(v[i] / scale);
                t = t > 127.0f ? 127.0f : t;
                t = t < -128.0f ? -128.0f : t;
                q[r * I + i] = (int8_t)t;
            }
        } else {
            for (int64_t i = 0; i < I; ++i) {
                float t;
                if (quant_per_channel)
                    t = v[i] / quant_scale[g * I + i] + (quant_offset ? quant_offset[g * I + i] : 0.0f);
                else
                    t = v[i] * (1.0f / quant_scale[g]) + (quant_offset ? quant_offset[g] : 0.0f);
                t = rintf(t);
                t = t > 127.0f ? 127.0f : t;
                t = t < -128.0f ? -128.0f : t;
                q[r * I + i] = (int8_t)t;
            }
        }
    }
    free(v);
    return 0;
}

/*
 * Activations other than SiLU.  The reference runs them unfused: gate_up product dequantised to the hidden dtype,
 * the activation on that 16-bit tensor, npu_dynamic_quant, down product
 * (vllm_ascend/ops/fused_moe/moe_mlp.py:484-549):
 *   gelu / gelu_tanh  F.gelu(gate, approximate=...) * up                                   (moe_mlp.py:516-520)
 *   swiglustep        silu(gate).clamp(max=L) * up.clamp(-L, L), L = swiglu_limit or 7     (moe_mlp.py:512-515,
 *                     vllm_ascend/ops/activation.py:63-86)
 *   swigluoai         g = gate.clamp(max=L), u = up.clamp(-L, L): g * sigmoid(alpha * g) * (u + beta)
 *                     (moe_mlp.py:123-137, 521-538)
 * [fixed by build] the activation is evaluated in fp32 on the 16-bit inputs and rounded ONCE to the hidden dtype
 * (torch would round after every operator; the reference's Triton / torch_npu kernels for these are closed or
 * compute in fp32 too -- PARITY UNPINNED), with erf by Abramowitz & Stegun 7.1.26 and tanh(z) = 1 - 2 / (1 +
 * exp(2 z)) on the shared exp; then the dynamic quantiser of orc_dynamic_quant on the rounded values.
 * h [rows, N] in the hidden dtype (gate = first half); q [rows, N/2] int8; qs [rows].
 */
ORC_API float orc_erff(float x)
{
    const float ax = fabsf(x);
    const float t = 1.0f / (1.0f + 0.3275911f * ax);
    float p = 1.061405429f;
    p = fmaf(p, t, -1.453152027f);
    p = fmaf(p, t, 1.421413741f);
    p = fmaf(p, t, -0.284496736f);
    p = fmaf(p, t, 0.254829592f);
    const float y = 1.0f - (p * t) * orc_expf(-(ax * ax));
    return copysignf(y, x);
}

ORC_API float orc_tanhf(float z) { return 1.0f - 2.0f / (1.0f + orc_expf(2.0f * z)); }

enum { ORC_ACT_GELU = 1, ORC_ACT_GELU_TANH = 2, ORC_ACT_SWIGLUSTEP = 3, ORC_ACT_SWIGLUOAI = 4 };

static inline float act_mul(float g, float u, int act, float limit, float alpha, float beta)
{
    if (act == ORC_ACT_GELU) return ((0.5f * g) * (1.0f + orc_erff(g * 0.70710678f))) * u;
    if (act == ORC_ACT_GELU_TANH) {
        const float inner = 0.7978845608f * (g + 0.044715f * ((g * g) * g));
        return ((0.5f * g) * (1.0f + orc_tanhf(inner))) * u;
    }
    if (act == ORC_ACT_SWIGLUSTEP) {
        float s = g / (1.0f + orc_expf(-g));
        s = s > limit ? limit : s;
        u = u > limit ? limit : u;
        u = u < -limit ? -limit : u;
        return s * u;
    }
    if (limit > 0.0f) {
        g = g > limit ? limit : g;
        u = u > limit ? limit : u;
        u = u < -limit ? -limit : u;
    }
    return (g * (1.0f / (1.0f + orc_expf(-(alpha * g))))) * (u + beta);
}

ORC_API int orc_act_mul_quant(const uint16_t *h, int64_t rows, int64_t N, int act, float limit, float alpha,
                              float beta, int8_t *q, float *qs)
{
    if (act < ORC_ACT_GELU || act > ORC_ACT_SWIGLUOAI) return -1;
    const int64_t I = N / 2;
#pragma omp parallel
    {
        float *y = (float *)malloc(sizeof(float) * (size_t)I);
#pragma omp for
        for (int64_t r = 0; r < rows; ++r) {
            float a = 0.0f;
            for (int64_t i = 0; i < I; ++i) {
                const float v = h2f(f2h(act_mul(h2f(h[r * N + i]), h2f(h[r * N + I + i]), act, limit, alpha, beta)));
                y[i] = v;
                const float b = fabsf(v);
                a = b > a ? b : a;
            }
            const float s = a / 127.0f;
            qs[r] = a == 0.0f ? 0.0f : s;
            for (int64_t i = 0; i < I; ++i) {
                float t = a == 0.0f ? 0.0f : rintf(y[i] / s);
                t = t > 127.0f ? 127.0f : t;
                t = t < -128.0f ? -128.0f : t;
                q[r * I + i] = (int8_t)t;
            }
        }
        free(y);
    }
    return 0;
}

/*
 * W4A8 down projection tail:  o[r,n] = bf16( (f[r,n] + bias[e,n]) * s1[r] ), f from orc_gmm_w4_grouped.
 * (the token scale is applied last, as in the reference's A8W4 kernel,
 * csrc/gmm/grouped_matmul_swiglu_quant/op_kernel/grouped_matmul_swiglu_quant_a8w4_msd_post.h).
 */
ORC_API int orc_w4_rows_to_bf16(const float *f, const float *s1, int64_t rows, int64_t N, uint16_t *o)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t n = 0; n < N; ++n) o[r * N + n] = f2h(f[r * N + n] * s1[r]);
    return 0;
}

/* ------------------------------------------------------------------ router gate
 * logits = x.float() @ W.T in fp32: AscendGateLinear.forward (vllm_ascend/ops/fused_moe/gate_linear.py:55-63)
 * and the internal-router branch of the layer (vllm_ascend/ops/fused_moe/fused_moe.py:264-271); both end in
 * F.linear, whose summation order belongs to the BLAS behind it.  [fixed by build]: K in chunks of 128; inside
 * a chunk acc = fmaf(x_k, w_k, acc) for ascending k from +0; chunk results are added in ascending order to a
 * total that starts at +0; the bias, when present, is added last.  fmaf here is the correctly rounded fused
 * multiply-add of C99 (an explicit call, not a contraction).
 * x_is_bf16: x holds bf16 bit patterns (uint16), else float. */
ORC_API void orc_router_gate(const void *x, int x_is_bf16, const float *w, const float *bias, int64_t T, int64_t H,
                             int64_t E, float *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        float *xf = (float *)malloc((size_t)H * sizeof(float));
        for (int64_t k = 0; k < H; ++k)
            xf[k] = x_is_bf16 ? h2f(((const uint16_t *)x)[t * H + k]) : ((const float *)x)[t * H + k];
        for (int64_t e = 0; e < E; ++e) {
            const float *we = w + e * H;
            float total = 0.0f;
            for (int64_t k0 = 0; k0 < H; k0 += 128) {
                const int64_t k1 = k0 + 128 < H ? k0 + 128 : H;
                float acc = 0.0f;
                for (int64_t k = k0; k < k1; ++k) acc = fmaf(xf[k], we[k], acc);
                total = total + acc;
            }
            out[t * E + e] = bias ? total + bias[e] : total;
        }
        free(xf);
    }
}

/* --- small conversion exports used by the Python wrapper ------------------- */

ORC_API void orc_f32_to_bf16(const float *in, int64_t n, uint16_t *out)
{
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16(in[i]);
}

ORC_API void orc_bf16_to_f32(const uint16_t *in, int64_t n, float *out)
{
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_f32(in[i]);
}

ORC_API void orc_f32_to_f16(const float *in, int64_t n, uint16_t *out)
{
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_f16(in[i]);
}

ORC_API void orc_f16_to_f32(const uint16_t *in, int64_t n, float *out)
{
    for (int64_t i = 0; i < n; ++i) out[i] = f16_to_f32(in[i]);
}

ORC_API int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
