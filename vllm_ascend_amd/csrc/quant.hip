// Per-token dynamic int8 quantisation and the int32 -> SwiGLU -> int8 split op.
//
// One workgroup (256 lanes = 4 wavefronts) per row.  The row absmax is reduced
// with wavefront shuffles, then across the four wavefronts through LDS; the
// row is read twice (the second read hits L2) in 16-byte vectors.
#include <type_traits>

#include "moe355_common.h"

namespace moe355 {

__device__ __forceinline__ float block_max_256(float v, float* lds4)
{
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    float m = lds4[0];
    m = lds4[1] > m ? lds4[1] : m;
    m = lds4[2] > m ? lds4[2] : m;
    m = lds4[3] > m ? lds4[3] : m;
    __syncthreads();
    return m;
}

// x [rows, cols] bf16 or fp16 (DT) -> q int8, scale fp32.  VEC: cols % 8 == 0 and 16-byte aligned rows.
// NV > 0 (VEC only): rows of at most NV x 2048 values stay in registers between the two passes.
template <bool VEC, int DT, int NV = 0>
__global__ __launch_bounds__(256) void dynamic_quant_kernel(const uint16_t* __restrict__ x, int64_t cols,
                                                                 int8_t* __restrict__ q, float* __restrict__ scale,
                                                                 int ieee_only)
{
    __shared__ float lds4[4];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * cols;
    int8_t* qr = q + row * cols;
    float a = 0.0f;
    if constexpr (VEC && NV > 0) {
        const int64_t nv = cols >> 3;
        const v8u16* xv = (const v8u16*)xr;
        v8u16 held[NV];
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            const int64_t i = threadIdx.x + 256 * n;
            held[n] = i < nv ? xv[i] : (v8u16){0, 0, 0, 0, 0, 0, 0, 0};
        }
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float f = __builtin_fabsf(half_to_f32<DT>(held[n][j]));
                a = f > a ? f : a;
            }
        a = block_max_256(a, lds4);
        const float s = a / 127.0f;
        const RowDivisor d = row_divisor(s, ieee_only != 0);
        if (threadIdx.x == 0) scale[row] = (a == 0.0f) ? 0.0f : s;
        uint2* qv = (uint2*)qr;
        auto emit = [&](auto fast) {
#pragma unroll
            for (int n = 0; n < NV; ++n) {
                const int64_t i = threadIdx.x + 256 * n;
                uint32_t w[2] = {0u, 0u};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int8_t b = (a == 0.0f) ? (int8_t)0
                                           : quantise_by_row<decltype(fast)::value>(half_to_f32<DT>(held[n][j]), d);
                    w[j >> 2] |= (uint32_t)(uint8_t)b << (8 * (j & 3));
                }
                if (i < nv) qv[i] = make_uint2(w[0], w[1]);
            }
        };
        if (d.fast) emit(std::true_type{});
        else emit(std::false_type{});
        return;
    }
    if constexpr (VEC) {
        const int64_t nv = cols >> 3;
        const v8u16* xv = (const v8u16*)xr;
        for (int64_t i = threadIdx.x; i < nv; i += 256) {
            v8u16 v = xv[i];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float f = __builtin_fabsf(half_to_f32<DT>(v[j]));
                a = f > a ? f : a;
            }
        }
    } else {
        for (int64_t i = threadIdx.x; i < cols; i += 256) {
            float f = __builtin_fabsf(half_to_f32<DT>(xr[i]));
            a = f > a ? f : a;
        }
    }
    a = block_max_256(a, lds4);
    const float s = a / 127.0f;
    const RowDivisor d = row_divisor(s, ieee_only != 0);
    if (threadIdx.x == 0) scale[row] = (a == 0.0f) ? 0.0f : s;
    auto emit = [&](auto fast) {
        constexpr bool F = decltype(fast)::value;
        if constexpr (VEC) {
            const int64_t nv = cols >> 3;
            const v8u16* xv = (const v8u16*)xr;
            uint2* qv = (uint2*)qr;
            for (int64_t i = threadIdx.x; i < nv; i += 256) {
                v8u16 v = xv[i];
                uint32_t w[2] = {0u, 0u};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int8_t b = (a == 0.0f) ? (int8_t)0 : quantise_by_row<F>(half_to_f32<DT>(v[j]), d);
                    w[j >> 2] |= (uint32_t)(uint8_t)b << (8 * (j & 3));
                }
                qv[i] = make_uint2(w[0], w[1]);
            }
        } else {
            for (int64_t i = threadIdx.x; i < cols; i += 256)
                qr[i] = (a == 0.0f) ? (int8_t)0 : quantise_by_row<F>(half_to_f32<DT>(xr[i]), d);
        }
    };
    if (d.fast) emit(std::true_type{});
    else emit(std::false_type{});
}

// x [rows, n] int32 -> dequant (weight scale, then activation scale) -> SwiGLU -> dynamic int8.
// NH > 0: a thread keeps its (at most NH) SwiGLU values between the absmax and the rounding pass;
// NH == 0: any row length, the values are computed again in the second pass.
// alpha, beta: the SwiGLU of swiglu_mode 1, (u + beta) * g / (1 + exp(-alpha g)) on the clamped values.  form_b: the
// quantiser of the reference's grouped kernel class, which also runs every swiglu_mode 1 call on int32 x
// (scale = max * (float)(1.0 / 127.0), q = rint(v / scale)); otherwise scale = max / 127, q = rint(v * (1 / scale)).
template <int NH>
__global__ __launch_bounds__(256) void dequant_swiglu_quant_kernel(const int32_t* __restrict__ x,
                                                                   const float* __restrict__ w_scale,
                                                                   const float* __restrict__ a_scale, int64_t n,
                                                                   int activate_left, float limit, float alpha,
                                                                   float beta, int form_b,
                                                                   int8_t* __restrict__ y, float* __restrict__ scale)
{
    __shared__ float lds4[4];
    const int64_t row = blockIdx.x;
    const int64_t half = n >> 1;
    const int32_t* xr = x + row * n;
    const float as = a_scale[row];
    const int64_t goff = activate_left ? 0 : half;
    const int64_t uoff = activate_left ? half : 0;
    const bool plain = alpha == 1.0f && beta == 0.0f;  // the proven short SiLU covers exactly this case
    auto value = [&](int64_t i) {
        float g = ((float)xr[goff + i] * w_scale[goff + i]) * as;
        float u = ((float)xr[uoff + i] * w_scale[uoff + i]) * as;
        if (limit > 0.0f) {
            g = g > limit ? limit : g;
            u = u > limit ? limit : u;
            u = u < -limit ? -limit : u;
        }
        if (plain) return m_silu(g) * u;
        return (u + beta) * (g / (1.0f + m_expf(g * -alpha)));
    };
    float held[NH > 0 ? NH : 1];
    float a = 0.0f;
    if constexpr (NH > 0) {
#pragma unroll
        for (int j = 0; j < NH; ++j) {
            const int64_t i = threadIdx.x + 256 * j;
            held[j] = i < half ? value(i) : 0.0f;
            const float v = __builtin_fabsf(held[j]);
            a = v > a ? v : a;
        }
    } else {
        for (int64_t i = threadIdx.x; i < half; i += 256) {
            const float v = __builtin_fabsf(value(i));
            a = v > a ? v : a;
        }
    }
    a = block_max_256(a, lds4);
    const float s = form_b ? a * (float)(1.0 / 127.0) : a / 127.0f;
    const float inv = 1.0f / s;
    if (threadIdx.x == 0) scale[row] = (a == 0.0f) ? 0.0f : s;
    int8_t* yr = y + row * half;
    auto quantise = [&](float v) { return (a == 0.0f) ? (int8_t)0 : sat_rint_i8(form_b ? v / s : v * inv); };
    if constexpr (NH > 0) {
#pragma unroll
        for (int j = 0; j < NH; ++j) {
            const int64_t i = threadIdx.x + 256 * j;
            if (i < half) yr[i] = quantise(held[j]);
        }
    } else {
        for (int64_t i = threadIdx.x; i < half; i += 256) yr[i] = quantise(value(i));
    }
}

// Static quantisation mode of the op above: q = rint(y / quant_scale[c] + quant_offset[c]) (one scale per output
// channel) or rint(y * (1 / quant_scale[0]) + quant_offset[0]) (one scale), saturated; no scale output.
__global__ __launch_bounds__(256) void dequant_swiglu_quant_static_kernel(
    const int32_t* __restrict__ x, const float* __restrict__ w_scale, const float* __restrict__ a_scale,
    const float* __restrict__ q_scale, int per_channel, const float* __restrict__ q_offset, int64_t n,
    int activate_left, float limit, int8_t* __restrict__ y)
{
    const int64_t row = blockIdx.x;
    const int64_t half = n >> 1;
    const int32_t* xr = x + row * n;
    const float as = a_scale[row];
    const int64_t goff = activate_left ? 0 : half;
    const int64_t uoff = activate_left ? half : 0;
    const float inv0 = 1.0f / q_scale[0];
    for (int64_t i = threadIdx.x; i < half; i += 256) {
        float g = ((float)xr[goff + i] * w_scale[goff + i]) * as;
        float u = ((float)xr[uoff + i] * w_scale[uoff + i]) * as;
        if (limit > 0.0f) {
            g = g > limit ? limit : g;
            u = u > limit ? limit : u;
            u = u < -limit ? -limit : u;
        }
        const float v = m_silu(g) * u;
        float t;
        if (per_channel) t = v / q_scale[i] + (q_offset ? q_offset[i] : 0.0f);
        else t = v * inv0 + (q_offset ? q_offset[0] : 0.0f);
        y[row * half + i] = sat_rint_i8(t);
    }
}

// The general form of the op above: rows in groups (group_index = row counts) with a weight scale, bias and quant
// scale per group, an int32 bias added to x or a float bias added after the scales, no activation scale, and the
// clamped / scaled SwiGLU of swiglu_mode 1 (csrc/moe/dequant_swiglu_quant/op_kernel/dequant_swiglu_quant.h:211-242,
// 380-424, 627-677).  Its dynamic quantiser multiplies the row maximum by (float)(1.0 / 127.0) and divides the
// values by that scale (:681-738).  One workgroup per row; the first wavefront finds the row's group from the
// counts.  Rows past the last group get y = 0 and scale = 0.
struct DsqArgs {
    const int32_t* x;
    const float* w_scale;
    const float* a_scale;
    const void* bias;
    int bias_kind;  // 0 none, 1 int32, 2 float
    const int64_t* group_index;
    int num_groups;
    int64_t n;
    int activate_left, swiglu_mode;
    float limit, alpha, beta;
    int quant_mode;
    const float* q_scale;
    int q_per_channel;
    const float* q_offset;
    int8_t* y;
    float* scale;
};

__global__ __launch_bounds__(256) void dequant_swiglu_quant_grouped_kernel(DsqArgs a)
{
    __shared__ float lds4[4];
    __shared__ int s_group;
    const int64_t row = blockIdx.x;
    const int64_t half = a.n >> 1;
    int g = 0;
    if (a.group_index) {
        if (threadIdx.x < 64) {
            const int lane = threadIdx.x;
            const int per = (a.num_groups + 63) / 64;
            int64_t local = 0;
            for (int j = 0; j < per; ++j) {
                const int gg = lane * per + j;
                const int64_t c = gg < a.num_groups ? a.group_index[gg] : 0;
                local += c < 0 ? 0 : c;
            }
            int64_t incl = local;
            for (int off = 1; off < 64; off <<= 1) {
                const int64_t t = __shfl_up(incl, off, 64);
                if (lane >= off) incl += t;
            }
            int64_t start = incl - local;
            if (row >= start && row < incl) {
                for (int j = 0; j < per; ++j) {
                    const int gg = lane * per + j;
                    const int64_t c = gg < a.num_groups ? a.group_index[gg] : 0;
                    const int64_t cc = c < 0 ? 0 : c;
                    if (row < start + cc) {
                        s_group = gg;
                        break;
                    }
                    start += cc;
                }
            }
            if (lane == 63 && row >= incl) s_group = -1;
        }
        __syncthreads();
        g = s_group;
    }
    int8_t* yr = a.y + row * half;
    if (g < 0) {
        for (int64_t i = threadIdx.x; i < half; i += 256) yr[i] = 0;
        if (threadIdx.x == 0 && a.scale) a.scale[row] = 0.0f;
        return;
    }
    const int32_t* xr = a.x + row * a.n;
    const float* ws = a.w_scale + (int64_t)g * a.n;
    const int64_t aoff = a.activate_left ? 0 : half;
    const int64_t loff = a.activate_left ? half : 0;
    const float as = a.a_scale ? a.a_scale[row] : 1.0f;
    auto value = [&](int64_t i) {
        int32_t xa = xr[aoff + i], xl = xr[loff + i];
        if (a.bias_kind == 1) {
            const int32_t* b = (const int32_t*)a.bias + (int64_t)g * a.n;
            xa = (int32_t)((uint32_t)xa + (uint32_t)b[aoff + i]);
            xl = (int32_t)((uint32_t)xl + (uint32_t)b[loff + i]);
        }
        float act = (float)xa * ws[aoff + i], lin = (float)xl * ws[loff + i];
        if (a.a_scale) {
            act = act * as;
            lin = lin * as;
        }
        if (a.bias_kind == 2) {
            const float* b = (const float*)a.bias + (int64_t)g * a.n;
            act = act + b[aoff + i];
            lin = lin + b[loff + i];
        }
        float e;
        if (a.swiglu_mode == 1) {
            if (a.limit > 0.0f) {
                lin = lin > a.limit ? a.limit : lin;
                lin = lin < -a.limit ? -a.limit : lin;
            }
            lin = lin + a.beta;
            if (a.limit > 0.0f) act = act > a.limit ? a.limit : act;
            e = m_expf(act * -a.alpha);
        } else {
            e = m_expf(act * -1.0f);
        }
        return lin * (act / (1.0f + e));
    };
    if (a.quant_mode == 1) {
        float amax = 0.0f;
        for (int64_t i = threadIdx.x; i < half; i += 256) {
            const float v = __builtin_fabsf(value(i));
            amax = v > amax ? v : amax;
        }
        amax = block_max_256(amax, lds4);
        const float s = amax * (float)(1.0 / 127.0);
        if (threadIdx.x == 0) a.scale[row] = (amax == 0.0f) ? 0.0f : s;
        for (int64_t i = threadIdx.x; i < half; i += 256)
            yr[i] = (amax == 0.0f) ? (int8_t)0 : sat_rint_i8(value(i) / s);
    } else {
        for (int64_t i = threadIdx.x; i < half; i += 256) {
            const float v = value(i);
            float t;
            if (a.q_per_channel) {
                const int64_t c = (int64_t)g * half + i;
                t = v / a.q_scale[c] + (a.q_offset ? a.q_offset[c] : 0.0f);
            } else {
                t = v * (1.0f / a.q_scale[g]) + (a.q_offset ? a.q_offset[g] : 0.0f);
            }
            yr[i] = sat_rint_i8(t);
        }
    }
}

// erf by Abramowitz & Stegun 7.1.26 on the shared exp (absolute error below 5e-7 in fp32); the CPU checker runs the
// same operation sequence.
__device__ __forceinline__ float m_erff(float x)
{
    const float ax = __builtin_fabsf(x);
    const float t = 1.0f / (1.0f + 0.3275911f * ax);
    float p = 1.061405429f;
    p = __builtin_fmaf(p, t, -1.453152027f);
    p = __builtin_fmaf(p, t, 1.421413741f);
    p = __builtin_fmaf(p, t, -0.284496736f);
    p = __builtin_fmaf(p, t, 0.254829592f);
    const float y = 1.0f - (p * t) * m_expf(-(ax * ax));
    return __builtin_copysignf(y, x);
}

__device__ __forceinline__ float m_tanhf(float z) { return 1.0f - 2.0f / (1.0f + m_expf(2.0f * z)); }

enum { ACT_GELU = 1, ACT_GELU_TANH = 2, ACT_SWIGLUSTEP = 3, ACT_SWIGLUOAI = 4 };

template <int ACT>
__device__ __forceinline__ float act_mul(float g, float u, float limit, float alpha, float beta)
{
    if constexpr (ACT == ACT_GELU) {
        return ((0.5f * g) * (1.0f + m_erff(g * 0.70710678f))) * u;
    } else if constexpr (ACT == ACT_GELU_TANH) {
        const float inner = 0.7978845608f * (g + 0.044715f * ((g * g) * g));
        return ((0.5f * g) * (1.0f + m_tanhf(inner))) * u;
    } else if constexpr (ACT == ACT_SWIGLUSTEP) {
        float sg = m_silu(g);
        sg = sg > limit ? limit : sg;
        u = u > limit ? limit : u;
        u = u < -limit ? -limit : u;
        return sg * u;
    } else {
        if (limit > 0.0f) {
            g = g > limit ? limit : g;
            u = u > limit ? limit : u;
            u = u < -limit ? -limit : u;
        }
        return (g * (1.0f / (1.0f + m_expf(-(alpha * g))))) * (u + beta);
    }
}

// h [rows, n] 16-bit (gate = first half) -> activation(gate) * up in fp32, rounded once to the 16-bit dtype ->
// per-row dynamic int8 (scale = absmax / 127, q = rint(v / scale)).  One workgroup per row; rows at or beyond the
// last group (gl given) are left untouched.
template <int ACT, int DT>
__global__ __launch_bounds__(256) void act_mul_quant_kernel(const uint16_t* __restrict__ h,
                                                            const int64_t* __restrict__ gl, int gl_type, int E,
                                                            int64_t n, float limit, float alpha, float beta,
                                                            int8_t* __restrict__ q, float* __restrict__ scale)
{
    __shared__ float lds4[4];
    const int64_t row = blockIdx.x;
    if (gl) {
        int64_t r0, total;
        expert_rows(gl, gl_type, E - 1, threadIdx.x & 63, r0, total);
        if (row >= total) return;
    }
    const int64_t half = n >> 1;
    const uint16_t* hr = h + row * n;
    auto value = [&](int64_t i) {
        const float v = act_mul<ACT>(half_to_f32<DT>(hr[i]), half_to_f32<DT>(hr[half + i]), limit, alpha, beta);
        return half_to_f32<DT>(f32_to_half<DT>(v));
    };
    float a = 0.0f;
    for (int64_t i = threadIdx.x; i < half; i += 256) {
        const float v = __builtin_fabsf(value(i));
        a = v > a ? v : a;
    }
    a = block_max_256(a, lds4);
    const float s = a / 127.0f;
    if (threadIdx.x == 0) scale[row] = (a == 0.0f) ? 0.0f : s;
    for (int64_t i = threadIdx.x; i < half; i += 256)
        q[row * half + i] = (a == 0.0f) ? (int8_t)0 : sat_rint_i8(value(i) / s);
}

// out[i] = silu(g[i]) by the kernels' instruction sequence (form 0) or by the IEEE quotient (form 1)
template <int FORM>
__global__ __launch_bounds__(256) void silu_f32_kernel(const float* __restrict__ g, float* __restrict__ out,
                                                       int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = FORM == 0 ? m_silu(g[i]) : m_silu_ieee(g[i]);
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe355_silu_f32(const float* g, float* out, int64_t n, int form, void* stream)
{
    if (n < 0 || (form != 0 && form != 1)) return MOE355_E_ARG;
    if (n == 0) return MOE355_OK;
    if (!g || !out) return MOE355_E_ARG;
    if ((n + 255) / 256 > 0x7fffffffLL) return MOE355_E_SHAPE;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (form == 0) hipLaunchKernelGGL(silu_f32_kernel<0>, grid, dim3(256), 0, (hipStream_t)stream, g, out, n);
    else hipLaunchKernelGGL(silu_f32_kernel<1>, grid, dim3(256), 0, (hipStream_t)stream, g, out, n);
    return launch_status();
}

static int dynamic_quant_impl(const void* x, int x_dtype, int64_t rows, int64_t cols, int8_t* q, float* scale,
                              int ieee_only, void* stream)
{
    if (rows < 0 || cols <= 0) return MOE355_E_ARG;
    if (rows == 0) return MOE355_OK;
    if (!x || !q || !scale) return MOE355_E_ARG;
    if (x_dtype != MOE355_DT_BF16 && x_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (rows > 0x7fffffffLL) return MOE355_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    const bool vec = (cols % 8 == 0) && (((uintptr_t)x & 15) == 0) && (((uintptr_t)q & 7) == 0);
#define MOE355_DQ(V_, D_)                                                                                      \
    hipLaunchKernelGGL((dynamic_quant_kernel<V_, D_>), dim3((unsigned)rows), dim3(256), 0, st, (const uint16_t*)x, \
                       cols, q, scale, ieee_only)
#define MOE355_DQH(D_, N_)                                                                                        \
    hipLaunchKernelGGL((dynamic_quant_kernel<true, D_, N_>), dim3((unsigned)rows), dim3(256), 0, st,                \
                       (const uint16_t*)x, cols, q, scale, ieee_only)
    if (x_dtype == MOE355_DT_BF16) {
        if (vec && cols <= 2048) MOE355_DQH(MOE355_DT_BF16, 1);
        else if (vec && cols <= 4096) MOE355_DQH(MOE355_DT_BF16, 2);
        else if (vec && cols <= 8192) MOE355_DQH(MOE355_DT_BF16, 4);
        else if (vec) MOE355_DQ(true, MOE355_DT_BF16);
        else MOE355_DQ(false, MOE355_DT_BF16);
    } else {
        if (vec && cols <= 2048) MOE355_DQH(MOE355_DT_F16, 1);
        else if (vec && cols <= 4096) MOE355_DQH(MOE355_DT_F16, 2);
        else if (vec && cols <= 8192) MOE355_DQH(MOE355_DT_F16, 4);
        else if (vec) MOE355_DQ(true, MOE355_DT_F16);
        else MOE355_DQ(false, MOE355_DT_F16);
    }
#undef MOE355_DQH
#undef MOE355_DQ
    return launch_status();
}

extern "C" int moe355_dynamic_quant(const void* x, int x_dtype, int64_t rows, int64_t cols, int8_t* q, float* scale,
                                    void* stream)
{
    return dynamic_quant_impl(x, x_dtype, rows, cols, q, scale, 0, stream);
}

extern "C" int moe355_dynamic_quant_form(const void* x, int x_dtype, int64_t rows, int64_t cols, int8_t* q,
                                         float* scale, int form, void* stream)
{
    if (form != 0 && form != 1) return MOE355_E_ARG;
    return dynamic_quant_impl(x, x_dtype, rows, cols, q, scale, form, stream);
}

static void launch_dsq(const int32_t* x, const float* weight_scale, const float* activation_scale, int64_t rows,
                       int64_t n, int activate_left, float limit, float alpha, float beta, int form_b, int8_t* y,
                       float* scale, void* stream)
{
#define MOE355_DSQ(NH_)                                                                                         \
    hipLaunchKernelGGL(dequant_swiglu_quant_kernel<NH_>, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, x, \
                       weight_scale, activation_scale, n, activate_left, limit, alpha, beta, form_b, y, scale)
    const int64_t half = n / 2;
    if (half <= 4 * 256) MOE355_DSQ(4);
    else if (half <= 16 * 256) MOE355_DSQ(16);
    else MOE355_DSQ(0);
#undef MOE355_DSQ
}

extern "C" int moe355_dequant_swiglu_quant(const int32_t* x, const float* weight_scale, const float* activation_scale,
                                           int64_t rows, int64_t n, int activate_left, float clamp_limit, int8_t* y,
                                           float* scale, void* stream)
{
    if (rows < 0 || n <= 0 || (n & 1)) return MOE355_E_ARG;
    if (rows == 0) return MOE355_OK;
    if (!x || !weight_scale || !activation_scale || !y || !scale) return MOE355_E_ARG;
    if (rows > 0x7fffffffLL) return MOE355_E_SHAPE;
    launch_dsq(x, weight_scale, activation_scale, rows, n, activate_left, clamp_limit, 1.0f, 0.0f, 0, y, scale, stream);
    return launch_status();
}

extern "C" int moe355_dequant_swiglu_quant_static(const int32_t* x, const float* weight_scale,
                                                  const float* activation_scale, const float* quant_scale,
                                                  int64_t quant_scale_len, const float* quant_offset, int64_t rows,
                                                  int64_t n, int activate_left, float clamp_limit, int8_t* y,
                                                  void* stream)
{
    if (rows < 0 || n <= 0 || (n & 1)) return MOE355_E_ARG;
    if (quant_scale_len != 1 && quant_scale_len != n / 2) return MOE355_E_SHAPE;
    if (rows == 0) return MOE355_OK;
    if (!x || !weight_scale || !activation_scale || !quant_scale || !y) return MOE355_E_ARG;
    if (rows > 0x7fffffffLL) return MOE355_E_SHAPE;
    hipLaunchKernelGGL(dequant_swiglu_quant_static_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, x,
                       weight_scale, activation_scale, quant_scale, quant_scale_len != 1 ? 1 : 0,
                       quant_offset, n, activate_left, clamp_limit, y);
    return launch_status();
}

extern "C" int moe355_dequant_swiglu_quant_grouped(const int32_t* x, const float* weight_scale,
                                                   const float* activation_scale, const void* bias, int bias_kind,
                                                   const int64_t* group_index, int num_groups, int64_t rows, int64_t n,
                                                   int activate_left, int swiglu_mode, float clamp_limit,
                                                   float glu_alpha, float glu_bias, int quant_mode,
                                                   const float* quant_scale, int64_t quant_scale_len,
                                                   const float* quant_offset, int8_t* y, float* scale, void* stream)
{
    if (rows < 0 || n <= 0 || (n & 1) || num_groups < 1) return MOE355_E_ARG;
    if (bias_kind < 0 || bias_kind > 2 || (bias_kind != 0) != (bias != nullptr)) return MOE355_E_ARG;
    if ((swiglu_mode != 0 && swiglu_mode != 1) || (quant_mode != 0 && quant_mode != 1)) return MOE355_E_ARG;
    if (!group_index && num_groups != 1) return MOE355_E_ARG;
    int per_channel = 0;
    if (quant_mode == 0) {
        if (!quant_scale) return MOE355_E_ARG;
        if (quant_scale_len == (int64_t)num_groups * (n / 2) && n / 2 != 1) per_channel = 1;
        else if (quant_scale_len != num_groups) return MOE355_E_SHAPE;
    } else if (quant_scale || quant_offset) {
        return MOE355_E_UNSUPPORTED;  // the smooth scale of the dynamic mode
    }
    if (rows == 0) return MOE355_OK;
    if (!x || !weight_scale || !y || (quant_mode == 1 && !scale)) return MOE355_E_ARG;
    if (rows > 0x7fffffffLL) return MOE355_E_SHAPE;
    if (!group_index && bias_kind == 0 && activation_scale && quant_mode == 1) {
        // the common call (shared expert): the row kernel that keeps its values in registers
        const bool m1 = swiglu_mode == 1;
        launch_dsq(x, weight_scale, activation_scale, rows, n, activate_left, m1 ? clamp_limit : 0.0f,
                   m1 ? glu_alpha : 1.0f, m1 ? glu_bias : 0.0f, 1, y, scale, stream);
        return launch_status();
    }
    DsqArgs a;
    a.x = x;
    a.w_scale = weight_scale;
    a.a_scale = activation_scale;
    a.bias = bias;
    a.bias_kind = bias_kind;
    a.group_index = group_index;
    a.num_groups = num_groups;
    a.n = n;
    a.activate_left = activate_left;
    a.swiglu_mode = swiglu_mode;
    a.limit = clamp_limit;
    a.alpha = glu_alpha;
    a.beta = glu_bias;
    a.quant_mode = quant_mode;
    a.q_scale = quant_scale;
    a.q_per_channel = per_channel;
    a.q_offset = quant_offset;
    a.y = y;
    a.scale = scale;
    hipLaunchKernelGGL(dequant_swiglu_quant_grouped_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, a);
    return launch_status();
}

extern "C" int moe355_act_mul_quant(const void* h, int h_dtype, const int64_t* group_list, int group_list_type,
                                    int num_experts, int64_t rows, int64_t n, int activation, float limit, float alpha,
                                    float beta, int8_t* q, float* scale, void* stream)
{
    if (rows < 0 || n <= 0 || (n & 1)) return MOE355_E_ARG;
    if (activation < ACT_GELU || activation > ACT_SWIGLUOAI) return MOE355_E_UNSUPPORTED;
    if (h_dtype != MOE355_DT_BF16 && h_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (group_list && (num_experts <= 0 || (group_list_type != MOE355_GL_CUMSUM && group_list_type != MOE355_GL_COUNT)))
        return MOE355_E_ARG;
    if (activation == ACT_SWIGLUSTEP && !(limit > 0.0f)) return MOE355_E_ARG;
    if (rows == 0) return MOE355_OK;
    if (!h || !q || !scale) return MOE355_E_ARG;
    if (rows > 0x7fffffffLL) return MOE355_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define MOE355_AMQ(A_, D_)                                                                                     \
    hipLaunchKernelGGL((act_mul_quant_kernel<A_, D_>), dim3((unsigned)rows), dim3(256), 0, st, (const uint16_t*)h, \
                       group_list, group_list_type, num_experts, n, limit, alpha, beta, q, scale)
#define MOE355_AMQ_D(A_)                                 \
    if (h_dtype == MOE355_DT_BF16) MOE355_AMQ(A_, MOE355_DT_BF16); \
    else MOE355_AMQ(A_, MOE355_DT_F16)
    if (activation == ACT_GELU) { MOE355_AMQ_D(ACT_GELU); }
    else if (activation == ACT_GELU_TANH) { MOE355_AMQ_D(ACT_GELU_TANH); }
    else if (activation == ACT_SWIGLUSTEP) { MOE355_AMQ_D(ACT_SWIGLUSTEP); }
    else { MOE355_AMQ_D(ACT_SWIGLUOAI); }
#undef MOE355_AMQ_D
#undef MOE355_AMQ
    return launch_status();
}
