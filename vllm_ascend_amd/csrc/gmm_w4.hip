// W4A8 grouped GEMM: int4 weights (two per byte), int8 activations, fp32 scales per K group.
//
// Weight-streaming kernel (the W4A8 shapes are HBM-bound: half the weight bytes of W8A8).
// Storage tile = 32 channels x 64 K in 1 KiB: lane l (channel l%32, K half l/32) holds 16 bytes;
// byte j carries, in its low nibble, w[k = 64*kb + 16*(l/32) + j] (first 32-wide K step) and in its
// high nibble w[k + 32] (second K step).  One 16-byte load therefore feeds two MFMAs.  A nibble is
// moved into the top half of its byte ((v << 4) & 0xF0..., v & 0xF0...), which is the signed int8
// value 16*w: the int32 accumulator is exactly 16x the true sum and is shifted back before use.
// Every `group` K values the accumulator is folded into fp32, f += float(acc) * scale[e, g, n], in
// ascending group order (one wavefront owns the whole K range of its channels, so the order is the
// sequential one), then f (+ bias) * token_scale goes through the shared epilogues.
#include <hip/hip_ext.h>

#include <type_traits>

#include "gmm_common.h"

namespace moe355 {

// ------------------------------------------------------------------ format cast
// SRC 0: int8 [E, N, K] holding one int4 value (-8..7) each (checkpoint order).
// SRC 1: packed [E, K, N/2] bytes, low nibble = even channel (the reference's packing,
//        vllm_ascend/quantization/methods/w4a8.py:327-336).
template <int SRC>
__global__ __launch_bounds__(256) void format_cast_nz_int4_kernel(const uint8_t* __restrict__ w, int64_t E, int64_t N,
                                                                  int64_t K, uint8_t* __restrict__ out)
{
    const int64_t total = E * N * K / 32;  // 16-byte chunks (32 nibbles each)
    const int64_t KB = K / 64, NB = N / 32;
    for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
        const int lane = (int)(id & 63);
        const int64_t tile = id >> 6;
        const int64_t kb = tile % KB;
        const int64_t nb = (tile / KB) % NB;
        const int64_t e = tile / (KB * NB);
        const int64_t n = nb * 32 + (lane & 31);
        const int64_t k0 = kb * 64 + (lane >> 5) * 16;
        uint32_t p[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            uint32_t lo, hi;
            if constexpr (SRC == 0) {
                lo = w[(e * N + n) * K + k0 + j] & 0xFu;
                hi = w[(e * N + n) * K + k0 + 32 + j] & 0xFu;
            } else {
                const uint8_t b0 = w[(e * K + k0 + j) * (N / 2) + (n >> 1)];
                const uint8_t b1 = w[(e * K + k0 + 32 + j) * (N / 2) + (n >> 1)];
                lo = (n & 1) ? (b0 >> 4) : (b0 & 0xFu);
                hi = (n & 1) ? (b1 >> 4) : (b1 & 0xFu);
            }
            p[j >> 2] |= (lo | (hi << 4)) << (8 * (j & 3));
        }
        *(v4i*)(out + id * 16) = (v4i){(int)p[0], (int)p[1], (int)p[2], (int)p[3]};
    }
}

// corr[e, n] = 8 * sum_g float(sum_{k in g} w[e, n, k]) * scale[e, g, n]  (g ascending, fp32):
// the term the Ascend kernel's unsigned-nibble trick adds (x = (x - 8) + 8), which callers of the
// int4 op pass in as `bias` / `weight_assist_matrix`.  One wavefront per (expert, 32-channel tile).
__global__ __launch_bounds__(256) void w4_offset_correction_kernel(const uint8_t* __restrict__ w4,
                                                                   const float* __restrict__ gscale, int E, int N,
                                                                   int K, int group, float* __restrict__ corr)
{
    const int lane = threadIdx.x & 63;
    const int64_t tile_row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int NB = N >> 5, KB64 = K >> 6;
    if (tile_row >= (int64_t)E * NB) return;
    const int e = (int)(tile_row / NB), nb = (int)(tile_row % NB);
    const uint8_t* wp = w4 + (tile_row * KB64) * 1024 + lane * 16;
    const int steps_per_group = group >> 6;
    const int n_groups = K / group;
    const int ch = nb * 32 + (lane & 31);
    float total = 0.0f;
    for (int g = 0; g < n_groups; ++g) {
        int sum = 0;
        for (int t = 0; t < steps_per_group; ++t) {
            const v4i v = *(const v4i*)(wp + (int64_t)(g * steps_per_group + t) * 1024);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
#pragma unroll
                for (int b = 0; b < 8; ++b) sum += ((int)((unsigned)v[d] << (28 - 4 * b))) >> 28;  // signed nibble b
            }
        }
        sum += __shfl_xor(sum, 32, 64);  // the two K halves of the tile
        total = total + (float)sum * gscale[((int64_t)e * n_groups + g) * N + ch];
    }
    if (lane < 32) corr[(int64_t)e * N + ch] = 8.0f * total;
}

struct W4Args {
    GmmArgs g;            // x, gl, R, K, N, E, row_scale, limit, outputs; g.w unused
    const uint8_t* w4;    // tiled int4 storage
    const float* gscale;  // [E, K/group, N]
    const float* bias;    // [E, N] or null, added before the token scale
    int group;            // K values per scale group (multiple of 64)
};

__device__ __forceinline__ v4i nib_lo(v4i v)
{
    return (v4i){(int)(((unsigned)v[0] << 4) & 0xF0F0F0F0u), (int)(((unsigned)v[1] << 4) & 0xF0F0F0F0u),
                 (int)(((unsigned)v[2] << 4) & 0xF0F0F0F0u), (int)(((unsigned)v[3] << 4) & 0xF0F0F0F0u)};
}
__device__ __forceinline__ v4i nib_hi(v4i v)
{
    return (v4i){(int)((unsigned)v[0] & 0xF0F0F0F0u), (int)((unsigned)v[1] & 0xF0F0F0F0u),
                 (int)((unsigned)v[2] & 0xF0F0F0F0u), (int)((unsigned)v[3] & 0xF0F0F0F0u)};
}

// Float twin of epilogue_run: g/u already hold sum_g float(acc_g)*scale_g (+ bias); the token scale is
// applied here, last.
template <int EPI>
__device__ __forceinline__ void epilogue_run_w4(const GmmArgs& a, int64_t row, bool valid, int c0, int c1,
                                                const float* g, const float* u, float rs)
{
    if (!valid) return;
    if constexpr (EPI == EPI_DEQUANT) {
        v4u16 o0, o1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o0[j] = a.out_f16 ? f32_to_f16(g[j] * rs) : f32_to_bf16(g[j] * rs);
            o1[j] = a.out_f16 ? f32_to_f16(u[j] * rs) : f32_to_bf16(u[j] * rs);
        }
        *(v4u16*)(a.out + row * a.N + c0) = o0;
        *(v4u16*)(a.out + row * a.N + c1) = o1;
    } else {
        const int I = a.N >> 1;
        v4f yv;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float gg = g[j] * rs;
            float uu = u[j] * rs;
            if (a.limit > 0.0f) {
                gg = gg > a.limit ? a.limit : gg;
                uu = uu > a.limit ? a.limit : uu;
                uu = uu < -a.limit ? -a.limit : uu;
            }
            yv[j] = m_silu(gg) * uu;
        }
        *(v4f*)(a.y + row * I + c0) = yv;
    }
}

// Chunk c of the list "rows of expert 0 in pieces of CHUNK rows, then expert 1, ...": which expert, which
// rows, and whether it is the expert's only chunk.  Every lane returns the same answer; false past the last chunk.  Lane l owns experts
// [l*seg, (l+1)*seg): local counts, a wavefront scan, then a short walk inside the owning lane's segment.
__device__ __forceinline__ bool find_chunk(const int64_t* gl, int gl_type, int E, int c, int CHUNK, int lane, int& e,
                                           int64_t& row0, int64_t& row1, bool& only_chunk)
{
    auto rows_of = [&](int i) -> int {
        const int64_t m = (gl_type == MOE355_GL_COUNT) ? gl[i] : gl[i] - (i > 0 ? gl[i - 1] : 0);
        return m < 0 ? 0 : (int)m;
    };
    const int seg = (E + 63) >> 6;
    const int e0 = lane * seg;
    int rows = 0, chunks = 0;
    for (int j = 0; j < seg; ++j) {
        if (e0 + j < E) {
            const int m = rows_of(e0 + j);
            rows += m;
            chunks += (m + CHUNK - 1) / CHUNK;
        }
    }
    int inc_rows = rows, inc_chunks = chunks;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int r = __shfl_up(inc_rows, off, 64), k = __shfl_up(inc_chunks, off, 64);
        if (lane >= off) {
            inc_rows += r;
            inc_chunks += k;
        }
    }
    if (c >= __shfl(inc_chunks, 63, 64)) return false;
    const uint64_t owns = __ballot(c < inc_chunks);  // lanes at or after the owner
    const int owner = __builtin_ctzll(owns);
    int cc = __shfl(inc_chunks - chunks, owner, 64);
    int64_t rr = __shfl(inc_rows - rows, owner, 64);
    const int oe0 = owner * seg;
    for (int j = 0; j < seg; ++j) {
        const int i = oe0 + j;
        if (i >= E) break;
        const int m = rows_of(i);
        const int nc = (m + CHUNK - 1) / CHUNK;
        if (c - cc < nc) {
            e = i;
            row0 = rr + (int64_t)(c - cc) * CHUNK;
            row1 = rr + m;
            only_chunk = nc == 1;
            return true;
        }
        cc += nc;
        rr += m;
    }
    return false;
}

// One wavefront per unit (chunk of up to 64 rows of one expert, pair of 32-channel tiles), whole K range in
// ascending order (the fp32 sum over scale groups has one fixed order).  An expert with many rows becomes
// many units that run side by side on different CUs and find the expert's weights in L2 / Infinity Cache,
// instead of one wavefront streaming the same weights once per 32 rows.
// The four wavefronts of a workgroup work on the same chunk (four neighbouring tile pairs), so the chunk's
// tokens go through LDS once per workgroup: every thread loads one 16-byte piece of the 64 x 64-byte K block
// (rows are read in 64-byte runs instead of 16-byte crumbs per lane), writes it in MFMA-operand order, and
// each wavefront reads its four B operands back with conflict-free 1 KiB sweeps.
constexpr int kW4Chunk = 64;
constexpr int kW4LdsGroups = 32;  // K groups whose scales are kept in LDS (8 KiB per wavefront)
// LDS_SCALES: the group scales of the wavefront's channels fit LDS (K / group <= kW4LdsGroups)
template <int EPI, bool LDS_SCALES>
__global__ __launch_bounds__(256, 2) void gmm_w4_stream_kernel(W4Args p)
{
    const GmmArgs& a = p.g;
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int NB = a.N >> 5, KB64 = a.K >> 6;
    const int upe = NB >> 1;
    // workgroup = (chunk, four neighbouring tile pairs); a wavefront past the last pair still stages tokens
    const int quads = (upe + 3) >> 2;
    const int chunk = (int)(blockIdx.x / quads);
    const int pi_raw = (int)(blockIdx.x % quads) * 4 + wave;
    const bool have = pi_raw < upe;
    const int pi = have ? pi_raw : 0;
    int e = 0;
    int64_t row0 = 0, row1 = 0;
    bool single_chunk = false;
    if (!find_chunk(a.gl, a.gl_type, a.E, chunk, kW4Chunk, lane, e, row0, row1, single_chunk)) return;
    if (row1 > a.R) row1 = a.R;
    if (row1 <= row0) return;
    const int nb0 = (EPI == EPI_SWIGLU) ? pi : 2 * pi;
    const int nb1 = (EPI == EPI_SWIGLU) ? pi + upe : 2 * pi + 1;

    const uint8_t* w0 = p.w4 + (((int64_t)e * NB + nb0) * KB64) * 1024 + lane * 16;
    const uint8_t* w1 = p.w4 + (((int64_t)e * NB + nb1) * KB64) * 1024 + lane * 16;
    // weights and tokens: rings of RW single K blocks, requested RW - 1 blocks ahead of their MFMAs.  Both
    // rings have the same depth on purpose: the memory counter retires loads in order, so waiting for a
    // token block that was requested late would also wait for every weight block requested before it.
    constexpr int RW = LDS_SCALES ? 6 : 5;  // scales read from memory inside the fold need the registers of one ring slot
    v4i a0[RW], a1[RW];
    // STREAM: the expert has a single chunk, nobody else reads these weights: non-temporal loads (the faster
    // pure stream).  Otherwise the sibling chunks of the expert run at the same time on the same XCD (their
    // workgroup numbers differ by a multiple of 16) and ordinary loads let them share one fetch in L2.
    auto load_weights = [&](auto stream, int slot, int kb) {
        const int k = kb < KB64 ? kb : KB64 - 1;  // past the end: a valid block that is never used
        if constexpr (decltype(stream)::value) {
            a0[slot] = __builtin_nontemporal_load((const v4i*)(w0 + (int64_t)k * 1024));
            a1[slot] = __builtin_nontemporal_load((const v4i*)(w1 + (int64_t)k * 1024));
        } else {
            a0[slot] = *(const v4i*)(w0 + (int64_t)k * 1024);
            a1[slot] = *(const v4i*)(w1 + (int64_t)k * 1024);
        }
    };

    const int tok = lane & 31;
    const int hi = lane >> 5;
    const int steps_per_group = p.group >> 6;  // 64-wide K blocks per scale group
    const int n_groups = a.K / p.group;
    const float* gs = p.gscale + (int64_t)e * n_groups * a.N;

    __shared__ __attribute__((aligned(16))) int8_t Bs[2][kW4Chunk * 64];  // two stages of 64 rows x 64 K bytes
    int64_t row[2];
    bool valid[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        row[b] = row0 + 32 * b + tok;
        valid[b] = row[b] < row1;
    }
    // staging: thread t carries row (t % 16) + 16 * (t / 64), 16-byte piece (t / 16) % 4 of the K block
    const int srow = (threadIdx.x & 15) + 16 * wave;
    const int skc = (threadIdx.x >> 4) & 3;
    int64_t sr = row0 + srow;
    if (sr > row1 - 1) sr = row1 - 1;  // rows past the chunk's end repeat its last row (never stored)
    if (a.row_src) sr = a.row_src[sr];  // the row's values lie in its token's row
    const int8_t* xs = a.x + sr * a.K + skc * 16;
    const int lds_off = ((((skc >> 1) * 2 + (srow >> 5)) * 64) + (skc & 1) * 32 + (srow & 31)) * 16;
    const bool two = row0 + 32 < row1;  // the second token block holds rows (wavefront-uniform)

    v16i c0[2], c1[2];
    float f0[2][16], f1[2][16];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        c0[b] = (v16i){0};
        c1[b] = (v16i){0};
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            f0[b][v] = 0.0f;
            f1[b][v] = 0.0f;
        }
    }
    // The scales of this wavefront's 64 channels for every K group sit in LDS (when they fit: up to 32
    // groups), loaded once up front: the K loop then has no load whose result is needed at once, and its
    // waits for weights and tokens stay partial.
    __shared__ float Ss[4][LDS_SCALES ? kW4LdsGroups * 64 : 1];
    if constexpr (LDS_SCALES) {
        const int ch = lane < 32 ? nb0 * 32 + lane : nb1 * 32 + (lane - 32);
        for (int g0 = 0; g0 < n_groups; g0 += 8) {  // eight loads in flight at a time
            float t[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) t[j] = gs[(int64_t)(g0 + j < n_groups ? g0 + j : n_groups - 1) * a.N + ch];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (g0 + j < n_groups) Ss[wave][(g0 + j) * 64 + lane] = t[j];
        }
    }
    int in_group = 0, grp = 0;
    // f += float(acc / 16) * scale[e, grp, channel]
    auto fold_with = [&](const v4f* s0, const v4f* s1) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if (b == 1 && !two) break;  // no rows in the second token block: its accumulators stay zero
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    f0[b][4 * q + j] = f0[b][4 * q + j] + (float)(c0[b][4 * q + j] >> 4) * s0[q][j];
                    f1[b][4 * q + j] = f1[b][4 * q + j] + (float)(c1[b][4 * q + j] >> 4) * s1[q][j];
                }
            c0[b] = (v16i){0};
            c1[b] = (v16i){0};
        }
        in_group = 0;
        ++grp;
    };
    auto fold = [&]() {
        v4f s0[4], s1[4];
        if constexpr (LDS_SCALES) {
            const float* sl = &Ss[wave][grp * 64 + 4 * hi];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                s0[q] = *(const v4f*)(sl + 8 * q);
                s1[q] = *(const v4f*)(sl + 32 + 8 * q);
            }
            fold_with(s0, s1);
        } else {
            const float* s = gs + (int64_t)grp * a.N + 4 * hi;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                s0[q] = *(const v4f*)(s + nb0 * 32 + 8 * q);
                s1[q] = *(const v4f*)(s + nb1 * 32 + 8 * q);
            }
            fold_with(s0, s1);
        }
    };
    // tokens: K block kb lives in LDS stage kb & 1; treg[(kb) % RW] carries block kb from its load (RW - 1
    // steps before its MFMAs) until it is written to LDS in the step before it is used
    auto load_tokens = [&](int kb) { return *(const v4i*)(xs + (int64_t)(kb < KB64 ? kb : KB64 - 1) * 64); };
    v4i treg[RW];
    treg[0] = load_tokens(0);
    *(v4i*)(&Bs[0][lds_off]) = treg[0];
#pragma unroll
    for (int i = 1; i < RW; ++i) treg[i] = load_tokens(i);
    __syncthreads();
    auto step = [&](auto stream, int slot, int kb) {  // one 64-wide K block; slot = kb % RW (compile time)
        v4i bl[2], bh[2];  // [token block]: K 0..31 / 32..63 of the block
        const int8_t* st = Bs[kb & 1];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            bl[b] = *(const v4i*)(st + ((0 * 2 + b) * 64 + lane) * 16);
            bh[b] = *(const v4i*)(st + ((1 * 2 + b) * 64 + lane) * 16);
        }
        *(v4i*)(&Bs[(kb + 1) & 1][lds_off]) = treg[(slot + 1) % RW];  // block kb + 1 (stage last read in step kb - 1)
        treg[slot] = load_tokens(kb + RW);   // block kb has left its register in the step before
        const v4i l0 = nib_lo(a0[slot]), h0 = nib_hi(a0[slot]);
        const v4i l1 = nib_lo(a1[slot]), h1 = nib_hi(a1[slot]);
        load_weights(stream, (slot + RW - 1) % RW, kb + RW - 1);  // the slot block kb - 1 has just left
        c0[0] = mfma_i8(l0, bl[0], c0[0]);
        c0[0] = mfma_i8(h0, bh[0], c0[0]);
        c1[0] = mfma_i8(l1, bl[0], c1[0]);
        c1[0] = mfma_i8(h1, bh[0], c1[0]);
        if (two) {
            c0[1] = mfma_i8(l0, bl[1], c0[1]);
            c0[1] = mfma_i8(h0, bh[1], c0[1]);
            c1[1] = mfma_i8(l1, bl[1], c1[1]);
            c1[1] = mfma_i8(h1, bh[1], c1[1]);
        }
        if (++in_group == steps_per_group) fold();
        __syncthreads();  // block kb + 1 is visible; nobody still reads block kb
    };
    // whole passes through the ring without a condition on kb; the remainder is peeled
    const int kb_full = (KB64 / RW) * RW;
    auto k_loop = [&](auto stream) {
#pragma unroll
        for (int i = 0; i < RW - 1; ++i) load_weights(stream, i, i);
        for (int kb = 0; kb < kb_full; kb += RW) {
#pragma unroll
            for (int i = 0; i < RW; ++i) step(stream, i, kb + i);
        }
#pragma unroll
        for (int i = 0; i < RW - 1; ++i)
            if (kb_full + i < KB64) step(stream, i, kb_full + i);
    };
    if (single_chunk) k_loop(std::true_type{});
    else k_loop(std::false_type{});
    if (!have) return;  // (after the last barrier)
    // both token scales are requested before the first store of the epilogue (a load placed behind a store
    // would wait for it: the memory counter retires in order)
    float rs_pre[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int64_t r = valid[b] ? row[b] : row0;
        rs_pre[b] = a.row_scale[a.row_src ? (int64_t)a.row_src[r] : r];
    }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        if (b == 1 && !two) break;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ch = 8 * q + 4 * hi;
            float g[4], u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[j] = f0[b][4 * q + j];
                u[j] = f1[b][4 * q + j];
            }
            if (p.bias) {
                const v4f bg = *(const v4f*)(p.bias + (int64_t)e * a.N + nb0 * 32 + ch);
                const v4f bu = *(const v4f*)(p.bias + (int64_t)e * a.N + nb1 * 32 + ch);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    g[j] = g[j] + bg[j];
                    u[j] = u[j] + bu[j];
                }
            }
            epilogue_run_w4<EPI>(a, row[b], valid[b], nb0 * 32 + ch, nb1 * 32 + ch, g, u, rs_pre[b]);
        }
    }
}

// workgroups: an upper bound of the number of 64-row chunks (known on the host without reading the group
// list) times the groups of four tile pairs
static int64_t w4_blocks(int64_t rows, int num_experts, int64_t n)
{
    // a chunk has at least one row: a decode batch of a few rows has a few chunks, not one per expert (a workgroup
    // that only finds its chunk missing still costs its dispatch)
    const int64_t by_experts = rows / kW4Chunk + num_experts;
    return (rows < by_experts ? rows : by_experts) * ((n / 64 + 3) / 4);
}

template <int EPI>
static void launch_w4(const W4Args& p, int64_t blocks, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1)
{
    const bool lds_scales = p.g.K / p.group <= kW4LdsGroups;
    auto kernel = lds_scales ? gmm_w4_stream_kernel<EPI, true> : gmm_w4_stream_kernel<EPI, false>;
    if (ev0 && ev1)
        hipExtLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, st, ev0, ev1, 0, p);
    else
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(256), 0, st, p);
}

static int check_w4(const void* x, const void* w, const float* scale, const int64_t* gl, int gl_type, int64_t rows,
                    int64_t k, int64_t n, int E, int64_t group)
{
    if (rows < 0 || k <= 0 || n <= 0 || E <= 0 || group <= 0) return MOE355_E_ARG;
    if (gl_type != MOE355_GL_CUMSUM && gl_type != MOE355_GL_COUNT) return MOE355_E_ARG;
    if (n % 64 != 0 || k % 64 != 0 || group % 64 != 0 || k % group != 0) return MOE355_E_SHAPE;
    if (rows >= 0x7fffffffLL || n >= 0x7fffffffLL || k >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (rows > 0 && (!x || !w || !scale || !gl)) return MOE355_E_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15) || ((uintptr_t)scale & 15)) return MOE355_E_SHAPE;
    return MOE355_OK;
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe355_format_cast_nz_int4(const uint8_t* w, int source, int64_t num_experts, int64_t n, int64_t k,
                                          uint8_t* out, void* stream)
{
    if (num_experts <= 0 || n <= 0 || k <= 0 || !w || !out) return MOE355_E_ARG;
    if (source != 0 && source != 1) return MOE355_E_ARG;
    if (n % 32 != 0 || k % 64 != 0) return MOE355_E_SHAPE;
    if ((uintptr_t)out & 15) return MOE355_E_SHAPE;
    const int64_t total = num_experts * n * k / 32;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipStream_t st = (hipStream_t)stream;
    if (source == 0)
        hipLaunchKernelGGL(format_cast_nz_int4_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, st, w, num_experts, n, k,
                           out);
    else
        hipLaunchKernelGGL(format_cast_nz_int4_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, w, num_experts, n, k,
                           out);
    return launch_status();
}

extern "C" int moe355_w4_offset_correction(const uint8_t* weight_nz4, const float* weight_scale, int64_t group_size,
                                           int num_experts, int64_t n, int64_t k, float* corr, void* stream)
{
    if (num_experts <= 0 || n <= 0 || k <= 0 || group_size <= 0 || !weight_nz4 || !weight_scale || !corr)
        return MOE355_E_ARG;
    if (n % 32 != 0 || k % 64 != 0 || group_size % 64 != 0 || k % group_size != 0) return MOE355_E_SHAPE;
    if ((uintptr_t)weight_nz4 & 15) return MOE355_E_SHAPE;
    const int64_t tiles = (int64_t)num_experts * (n / 32);
    hipLaunchKernelGGL(w4_offset_correction_kernel, dim3((unsigned)((tiles + 3) / 4)), dim3(256), 0,
                       (hipStream_t)stream, weight_nz4, weight_scale, num_experts, (int)n, (int)k, (int)group_size,
                       corr);
    return launch_status();
}

static int gmm1_w4_impl(const int8_t* x, const uint8_t* weight_nz4, const float* weight_scale, int64_t group_size,
                        const float* bias, const float* x_scale, const int64_t* group_list, int group_list_type,
                        int64_t rows, int64_t k, int64_t n, int num_experts, float swiglu_limit, int8_t* out,
                        float* out_scale, void* workspace, size_t workspace_bytes, void* stream,
                        const int32_t* row_src)
{
    int rc = check_w4(x, weight_nz4, weight_scale, group_list, group_list_type, rows, k, n, num_experts, group_size);
    if (rc != MOE355_OK) return rc;
    if (rows == 0) return MOE355_OK;
    if (!x_scale || !out || !out_scale) return MOE355_E_ARG;
    if (((uintptr_t)bias & 15) || ((uintptr_t)out & 3)) return MOE355_E_SHAPE;
    const size_t ybytes = ((size_t)rows * (size_t)(n / 2) * 4 + 255) & ~(size_t)255;
    if (!workspace || ((uintptr_t)workspace & 255) || workspace_bytes < ybytes) return MOE355_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    W4Args p = {};
    p.g.x = x;
    p.g.gl = group_list;
    p.g.gl_type = group_list_type;
    p.g.R = rows;
    p.g.K = (int)k;
    p.g.N = (int)n;
    p.g.E = num_experts;
    p.g.row_scale = x_scale;
    p.g.row_src = row_src;
    p.g.limit = swiglu_limit;
    p.g.y = (float*)workspace;
    p.w4 = weight_nz4;
    p.gscale = weight_scale;
    p.bias = bias;
    p.group = (int)group_size;
    const int64_t blocks = w4_blocks(rows, num_experts, n);
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    take_profile_events(ev0, ev1);
    launch_w4<EPI_SWIGLU>(p, blocks, st, ev0, ev1);
    launch_swiglu_requant(p.g.y, group_list, group_list_type, num_experts, rows, (int)(n / 2), out, out_scale, st);
    return launch_status();
}

extern "C" int moe355_gmm1_swiglu_quant_w4(const int8_t* x, const uint8_t* weight_nz4, const float* weight_scale,
                                           int64_t group_size, const float* bias, const float* x_scale,
                                           const int64_t* group_list, int group_list_type, int64_t rows, int64_t k,
                                           int64_t n, int num_experts, float swiglu_limit, int8_t* out,
                                           float* out_scale, void* workspace, size_t workspace_bytes, void* stream)
{
    return gmm1_w4_impl(x, weight_nz4, weight_scale, group_size, bias, x_scale, group_list, group_list_type, rows, k,
                        n, num_experts, swiglu_limit, out, out_scale, workspace, workspace_bytes, stream, nullptr);
}

extern "C" int moe355_gmm1_swiglu_quant_w4_gather(const int8_t* x, const float* x_scale, const int32_t* row_token,
                                                  const uint8_t* weight_nz4, const float* weight_scale,
                                                  int64_t group_size, const float* bias, const int64_t* group_list,
                                                  int group_list_type, int64_t rows, int64_t k, int64_t n,
                                                  int num_experts, float swiglu_limit, int8_t* out, float* out_scale,
                                                  void* workspace, size_t workspace_bytes, void* stream)
{
    if (rows > 0 && !row_token) return MOE355_E_ARG;
    return gmm1_w4_impl(x, weight_nz4, weight_scale, group_size, bias, x_scale, group_list, group_list_type, rows, k,
                        n, num_experts, swiglu_limit, out, out_scale, workspace, workspace_bytes, stream, row_token);
}

extern "C" int moe355_gmm2_dequant_w4(const int8_t* x, const uint8_t* weight_nz4, const float* scale,
                                      int64_t group_size, const float* bias, const float* per_token_scale,
                                      const int64_t* group_list, int group_list_type, int64_t rows, int64_t k,
                                      int64_t n, int num_experts, void* out, int out_dtype, void* stream)
{
    int rc = check_w4(x, weight_nz4, scale, group_list, group_list_type, rows, k, n, num_experts, group_size);
    if (rc != MOE355_OK) return rc;
    if (out_dtype != MOE355_DT_BF16 && out_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (rows == 0) return MOE355_OK;
    if (!per_token_scale || !out) return MOE355_E_ARG;
    if (((uintptr_t)bias & 15) || ((uintptr_t)out & 7)) return MOE355_E_SHAPE;
    W4Args p = {};
    p.g.x = x;
    p.g.gl = group_list;
    p.g.gl_type = group_list_type;
    p.g.R = rows;
    p.g.K = (int)k;
    p.g.N = (int)n;
    p.g.E = num_experts;
    p.g.row_scale = per_token_scale;
    p.g.out = (uint16_t*)out;
    p.g.out_f16 = out_dtype == MOE355_DT_F16;
    p.w4 = weight_nz4;
    p.gscale = scale;
    p.bias = bias;
    p.group = (int)group_size;
    const int64_t blocks = w4_blocks(rows, num_experts, n);
    launch_w4<EPI_DEQUANT>(p, blocks, (hipStream_t)stream, nullptr, nullptr);
    return launch_status();
}
