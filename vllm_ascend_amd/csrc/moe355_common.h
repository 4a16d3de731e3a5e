// Shared device helpers for the gfx950 MoE kernels.
//
// Arithmetic contract shared by every kernel: IEEE binary32, round to nearest
// even, no fused multiply-add except where one is written out (the library is
// compiled with -ffp-contract=off; exp() and the router gate use explicit fmaf).
// A CPU program executing the same operation sequence produces the same bits.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/moe355.h"

#define MOE355_WAVE 64

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short v8u16 __attribute__((ext_vector_type(8)));
typedef unsigned short v4u16 __attribute__((ext_vector_type(4)));

namespace moe355 {

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __uint_as_float(u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __float_as_uint(f); }

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// fp32 -> bf16, round to nearest even (gfx950 has the conversion in hardware: v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    __bf16 b = (__bf16)f;
    uint16_t h;
    __builtin_memcpy(&h, &b, 2);
    return h;
}

__device__ __forceinline__ float f16_to_f32(uint16_t h)
{
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

__device__ __forceinline__ uint16_t f32_to_f16(float f)
{
    // The empty statement pins f as an fp32 value in a register.  Without it the compiler folds a preceding
    // multiply or add into v_fma_mixlo_f16, which rounds the exact product once, to fp16: on values whose fp32
    // rounding lands on an fp16 tie that differs from rounding twice (first to fp32, then to fp16), and the
    // arithmetic here is defined on fp32 intermediates.
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

// 16-bit float of kind DT (MOE355_DT_BF16 or MOE355_DT_F16) <-> fp32; narrowing rounds to nearest even.
template <int DT>
__device__ __forceinline__ float half_to_f32(uint16_t h)
{
    if constexpr (DT == MOE355_DT_F16) return f16_to_f32(h);
    else return bf16_to_f32(h);
}
template <int DT>
__device__ __forceinline__ uint16_t f32_to_half(float f)
{
    if constexpr (DT == MOE355_DT_F16) return f32_to_f16(f);
    else return f32_to_bf16(f);
}

// exp(x): argument clamped to [-87, 88.72283] (result always normal or +inf; NaN counts as -87),
// n = rint(x*log2e), two-part ln2 reduction, degree-5 polynomial, exact scaling by 2^n.
// The multiply-adds of the reduction and the polynomial are explicit fused operations (one rounding each,
// v_fma_f32); a CPU program calling fmaf in the same places produces the same bits.
__device__ __forceinline__ float m_expf(float x)
{
    x = __builtin_amdgcn_fmed3f(x, -87.0f, 88.72283f);  // min(max(x, -87), 88.72283) in one instruction
    float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    float y = __builtin_fmaf(p, r2, r);
    y = y + 1.0f;
    return __builtin_ldexpf(y, (int)n);
}

// silu(g) = g / (1 + exp(-g)) with the IEEE quotient written out: the definition, and what the CPU checker
// computes.  The kernels run m_silu below; this form is kept for the test that compares the two on every
// binary32 input.
__device__ __forceinline__ float m_silu_ieee(float g) { return g / (1.0f + m_expf(-g)); }

// The same function of g, bit for bit on all 2^32 inputs (NaN in, NaN out), in seven instructions behind the
// exponential instead of the twelve of a general division.  The general sequence scales both operands into the
// range of the hardware reciprocal, refines the reciprocal, corrects the quotient twice and repairs the special
// cases; here the divisor d = 1 + E is known to lie in [1, 2^128), which leaves one hazard: v_rcp_f32 flushes
// results below 2^-126, i.e. for d > 2^126 (g < -87.3).  Negative g therefore divide by d / 4 (a power of two
// commutes with every rounding involved: c * (1 + E) rounds like 1 + E) and scale the quotient back, which is
// exact too since 4 g / d stays far from overflow when E > 1; non-negative g divide by d itself (4 g would
// overflow for g > 2^126, and g / 4 would lose bits of subnormal g).  With a divisor in [1/4, 2^126] the
// reciprocal is within one unit, q0 within two, and one residual correction gives the correctly rounded
// quotient for every g -- not by a general theorem (the correction step can miss in a tie-like case for some
// operand pairs) but because d is a function of g: the pairs that occur are 2^32 and a test runs them all.
// v_div_fixup_f32 restores the two cases the chain cannot get right, the sign of g = -0 and g = +-inf.
__device__ __forceinline__ float m_silu(float g)
{
    const float E = m_expf(-g);
    const float c = g < 0.0f ? 0.25f : 1.0f;
    const float ds = __builtin_fmaf(E, c, c);
    const float r = __builtin_amdgcn_rcpf(ds);
    const float q0 = g * r;
    const float e = __builtin_fmaf(-ds, q0, g);
    const float q1 = __builtin_fmaf(e, r, q0);
    return __builtin_amdgcn_div_fixupf(q1 * c, ds, g);
}

// clamp(rint(v), -128, 127) as int8
__device__ __forceinline__ int8_t sat_rint_i8(float v)
{
    float r = __builtin_rintf(v);
    r = r > 127.0f ? 127.0f : r;
    r = r < -128.0f ? -128.0f : r;
    return (int8_t)(int)r;
}

// The token quantiser on 16-bit inputs: int8(rint(x / s)) for the values x of a row and the row's s = amax / 127.
// The definition divides (torch_npu.npu_dynamic_quant as the reference calls it,
// vllm_ascend/ops/fused_moe/moe_mlp.py:211-214: x / scale, rounded, then rounded to an integer); a row shares its
// divisor, so the kernels take the reciprocal once per row and correct the product once: q0 = x r,
// q1 = q0 + r (x - s q0) with fused operations.  That is not the correctly rounded quotient for every pair of
// binary32 numbers, but here x is a bf16 or fp16 value with |x| <= amax and amax is one too: about 2^31 pairs per
// type, and a test runs all of them through this sequence and through the division and finds the same int8
// (without the clamp to [-128, 127], which |x| <= amax makes idle: the quotient stays within +-127.00001).
// Rows whose divisor lies outside [2^-100, 2^100] (bf16 rows of all but vanishing or of astronomic values, where
// the reciprocal or the residual would leave the normal range) divide.
struct RowDivisor {
    float s, r;
    bool fast;
};

__device__ __forceinline__ RowDivisor row_divisor(float s, bool ieee_only = false)
{
    RowDivisor d;
    d.s = s;
    d.r = 1.0f / s;
    d.fast = !ieee_only && s >= 0x1p-100f && s <= 0x1p100f;
    return d;
}

template <bool FAST>
__device__ __forceinline__ int8_t quantise_by_row(float x, const RowDivisor& d)
{
    if constexpr (FAST) {
        const float q0 = x * d.r;
        const float e = __builtin_fmaf(-d.s, q0, x);
        // |x| <= amax keeps the quotient within +-127.00001: nothing to clamp
        return (int8_t)(int)__builtin_rintf(__builtin_fmaf(e, d.r, q0));
    } else {
        return sat_rint_i8(x / d.s);
    }
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

// Butterfly sum: after the loop every lane holds the same value; the order of
// additions is part of the arithmetic contract (partial[l] + partial[l ^ off]).
__device__ __forceinline__ float wave_tree_sum(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
    return v;
}

// Integer sum over the wavefront with DPP row shifts and row broadcasts (no LDS traffic);
// every lane returns the total.
__device__ __forceinline__ int wave_sum_i32(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return __builtin_amdgcn_readlane(v, 63);
}

// Inclusive prefix sum over the wavefront (the same DPP steps: shifts inside rows of 16, then the row totals).
__device__ __forceinline__ int wave_scan_inclusive_i32(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
    return v;
}

// Exclusive prefix sum of v over the threads of a workgroup (thread order), and the total.  Every thread of
// the workgroup calls it; lds holds one int per wavefront (at most 16) and can be reused after the call.
__device__ __forceinline__ int block_scan_exclusive_i32(int v, int* lds, int& total)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = (blockDim.x + 63) >> 6;
    const int inc = wave_scan_inclusive_i32(v);
    if (lane == 63) lds[wave] = inc;
    __syncthreads();
    int before = 0, all = 0;
    for (int w = 0; w < nwaves; ++w) {
        const int t = lds[w];
        before += w < wave ? t : 0;
        all += t;
    }
    __syncthreads();
    total = all;
    return before + inc - v;
}

// "a ranks before b": larger value first, ties to the lower index.
__device__ __forceinline__ bool ranks_before(float va, int ia, float vb, int ib)
{
    if (va > vb) return true;
    if (va < vb) return false;
    return ia < ib;
}

template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i)
{
    if constexpr (DT == MOE355_DT_F32) return ((const float*)p)[i];
    if constexpr (DT == MOE355_DT_BF16) return bf16_to_f32(((const uint16_t*)p)[i]);
    return f16_to_f32(((const uint16_t*)p)[i]);
}

template <int DT>
__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v)
{
    if constexpr (DT == MOE355_DT_F32) ((float*)p)[i] = v;
    else if constexpr (DT == MOE355_DT_BF16) ((uint16_t*)p)[i] = f32_to_bf16(v);
    else ((uint16_t*)p)[i] = f32_to_f16(v);
}

// Row range [row0, row1) of expert e from a group list held as counts or as a
// running sum.  Called by one full wave; every lane returns the same pair.
__device__ __forceinline__ void expert_rows(const int64_t* gl, int gl_type, int e, int lane, int64_t& row0,
                                            int64_t& row1)
{
    if (gl_type == MOE355_GL_CUMSUM) {
        row0 = e > 0 ? gl[e - 1] : 0;
        row1 = gl[e];
    } else {
        int s = 0;
        for (int i = lane; i < e; i += 64) s += (int)gl[i];
        s = wave_sum_i32(s);
        row0 = s;
        row1 = s + gl[e];
    }
}

inline int launch_status()
{
    return hipGetLastError() == hipSuccess ? MOE355_OK : MOE355_E_LAUNCH;
}

}  // namespace moe355
