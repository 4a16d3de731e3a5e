// Grouped int8 x int8 -> int32 GEMM for the expert MLPs, with the three
// epilogues (raw int32, dequant+SwiGLU, dequant to bf16), the weight format
// cast, and the per-row re-quantisation that finishes the SwiGLU op.
//
// Weight-streaming kernel: few rows per expert (decode), where the time is the
// HBM stream of the weights.  Work unit = (expert, pair of 32-channel tiles).
// The weights of a unit are contiguous 1 KiB tiles along K and go straight from
// HBM into MFMA operand registers with one 16-byte load per lane (no LDS: each
// weight byte is used by exactly one wavefront).  The expert's tokens are
// processed 32 at a time as the MFMA's second operand.  With KSPLIT = 4 the
// four wavefronts of a workgroup split K and add their int32 partials through
// LDS (integer addition: exact, order free).
#include <hip/hip_ext.h>
#include <stdlib.h>
#include <string.h>

#include "gmm_common.h"
#include "gmm_tiled.h"

namespace moe355 {

// ------------------------------------------------------------------ format cast
template <int LAYOUT>
__global__ __launch_bounds__(256) void format_cast_nz_kernel(const int8_t* __restrict__ w, int64_t E, int64_t N,
                                                             int64_t K, int8_t* __restrict__ out)
{
    const int64_t total = E * N * K / 16;
    const int64_t KB = K / 32, NB = N / 32;
    for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
        const int lane = (int)(id & 63);
        const int64_t tile = id >> 6;
        const int64_t kb = tile % KB;
        const int64_t nb = (tile / KB) % NB;
        const int64_t e = tile / (KB * NB);
        const int64_t n = nb * 32 + (lane & 31);
        const int64_t k0 = kb * 32 + (lane >> 5) * 16;
        v4i v;
        if constexpr (LAYOUT == MOE355_W_ENK) {
            v = *(const v4i*)(w + (e * N + n) * K + k0);
        } else {
            uint32_t p[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int b = 0; b < 16; ++b)
                p[b >> 2] |= (uint32_t)(uint8_t)w[(e * K + k0 + b) * N + n] << (8 * (b & 3));
            v = {(int)p[0], (int)p[1], (int)p[2], (int)p[3]};
        }
        *(v4i*)(out + id * 16) = v;
    }
}

// ------------------------------------------------------------------ streaming GEMM
// SLABS: K is cut into gridDim.y slabs (the dense few-row int32 product only; reading gridDim costs every
// wavefront a scalar load in front of its first weight request, 4 us per launch of the decode down GEMM)
// EARLY: the first weight tiles are requested before the group list is read (decode batches: nearly every expert
// has rows, and the lookup hides behind the HBM latency).  A launch that covers only some of the experts of a
// large batch reads the group list first: a unit whose expert is empty or belongs to the other kernel of the call
// would otherwise fetch 32 KiB for nothing, times thousands of units.
// PAIRS: the rows of an expert are not a range of a sorted activation but the (token, slot) pairs that chose it,
// found here from the ids of all pairs (at most 1024: a decode batch).  The four wavefronts of a workgroup work on
// one expert (KSPLIT == 1: four units of it; the host picks that form only when the units of an expert come in
// fours), scan a quarter of the ids each and leave the expert's pairs, in ascending order, in LDS.  The routing
// launch in front of the GEMM then is gating and quantisation only: no sort, no hand-off between workgroups.
// the n-th expert (counting from 0) whose group has rows, or -1: every lane of the wavefront calls it and gets the
// same answer (64 experts per step: one load per lane, a ballot, a count of bits)
__device__ __forceinline__ int nth_expert_with_rows(const int64_t* gl, int gl_type, int E, int n, int lane)
{
    int seen = 0;
    for (int base = 0; base < E; base += 64) {
        const int e = base + lane;
        int64_t c = 0;
        if (e < E) c = (gl_type == 1) ? gl[e] : gl[e] - (e ? gl[e - 1] : 0);
        const unsigned long long m = __ballot(c > 0);
        const int pc = __popcll(m);
        if (n < seen + pc) {
            unsigned long long t = m;
            for (int i = n - seen; i > 0; --i) t &= t - 1;
            return base + __builtin_ctzll(t);
        }
        seen += pc;
    }
    return -1;
}

constexpr int kPairMax = 1024;

// REQ (pair order, down GEMM): the activation is still the fp32 SwiGLU output; the workgroup re-quantises the rows
// of its expert itself, 32 at a time, into LDS (row maximum through LDS atomics on the bit patterns, which order
// like the non-negative values; then rint(v * (1 / (max / 127))), the arithmetic of swiglu_requant_kernel) and the
// MFMA operands come from there: the re-quantisation launch and its int8 round trip disappear.  The eight
// workgroups of an expert each do it again for the expert's few rows, which is nothing next to a launch.
template <int EPI, int KSPLIT, int UN, int OCC, bool SLABS = false, bool EARLY = true, bool PAIRS = false,
          bool REQ = false>
__global__ __launch_bounds__(256, OCC) void gmm_stream_kernel(GmmArgs a)
{
    static_assert(KSPLIT == 1 || KSPLIT == 4, "workgroup barriers need all four wavefronts on one unit");
    static_assert(!PAIRS || (!SLABS && EARLY && EPI != EPI_I32), "pair order: the two GEMMs of a decode layer");
    static_assert(!REQ || (PAIRS && EPI == EPI_DEQUANT), "the re-quantisation sits in the pair-order down GEMM");
    extern __shared__ __attribute__((aligned(16))) int8_t qtile[];  // REQ: 32 rows of K + 16 bytes
    __shared__ uint32_t qmax[REQ ? 32 : 1];
    __shared__ float qscale[REQ ? 32 : 1];
    __shared__ int32_t red[(KSPLIT > 1) ? 32 * 64 : 1];
    __shared__ uint16_t plist[PAIRS ? kPairMax : 1];
    __shared__ int32_t pcount[4];
    __shared__ uint32_t pmap[PAIRS ? 64 : 1];  // one bit per expert (at most 2048) that has pairs
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int NB = a.N >> 5, KB = a.K >> 5;
    const int upe = NB >> 1;  // units per expert
    const int64_t unit = (KSPLIT == 1) ? (int64_t)blockIdx.x * 4 + wave : (int64_t)blockIdx.x;
    // pair order with fewer pairs than experts: the grid has a slot per pair instead of a place per expert (most
    // experts are idle, and a workgroup that only finds that out still costs its dispatch: 28,000 of them are
    // 150 us), and slot s belongs to the s-th expert that has pairs at all
    const int places = (PAIRS && a.pair_slots > 0) ? a.pair_slots : (!PAIRS && !EARLY && a.gl_slots > 0) ? a.gl_slots : a.E;
    if (unit >= (int64_t)places * upe) return;  // KSPLIT == 1: no barriers below; KSPLIT == 4: whole workgroup leaves
    int e = (int)(unit / upe);
    const int p = (int)(unit % upe);
    const int nb0 = (EPI == EPI_SWIGLU) ? p : 2 * p;
    const int nb1 = (EPI == EPI_SWIGLU) ? p + upe : 2 * p + 1;

    // K is cut into gridDim.y slabs (SLABS: the dense few-row product, whose workgroups store their int32 partial
    // sums to a plane per slab, or without scratch add them into a zeroed result with atomics: integer addition,
    // exact and order free), and a slab into KSPLIT pieces, one per wavefront
    const int ks = (KSPLIT == 1) ? 0 : wave;
    int slab_begin = 0, slab_end = KB;
    if constexpr (SLABS) {
        slab_begin = (int)(((int64_t)KB * blockIdx.y) / gridDim.y);
        slab_end = (int)(((int64_t)KB * (blockIdx.y + 1)) / gridDim.y);
    }
    const int kb_begin = slab_begin + ((slab_end - slab_begin) * ks) / KSPLIT;
    const int kb_end = slab_begin + ((slab_end - slab_begin) * (ks + 1)) / KSPLIT;

    // pair order: wavefront w scans pairs [w Q, (w + 1) Q), Q a multiple of 64 and at most 256.  The ids are
    // requested in front of the weights: answers come back in the order of the requests, and the list of the
    // expert's pairs (which the token loads wait for) should not queue behind the first weight tiles from HBM.
    const int Q = PAIRS ? (((int)a.R + 255) >> 8) << 6 : 0;
    int pid[PAIRS ? 4 : 1];
    if constexpr (PAIRS) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int f = wave * Q + c * 64 + lane;
            pid[c] = (c * 64 < Q && f < (int)a.R) ? a.pair_ids[f] : -1;
        }
    }
    if constexpr (PAIRS) {
        if (a.pair_slots > 0) {
            // the experts that have pairs, as a bit map in LDS; every wavefront then finds the expert of the
            // workgroup's slot by itself: a count of the bits in front of each word, and the word's bit
            if (threadIdx.x < 64) pmap[threadIdx.x] = 0u;
            __syncthreads();
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (pid[c] >= 0 && pid[c] < a.E) atomicOr(&pmap[pid[c] >> 5], 1u << (pid[c] & 31));
            __syncthreads();
            const uint32_t bits = pmap[lane];
            const int cnt = __popc(bits);
            int incl = cnt;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int t = __shfl_up(incl, off, 64);
                if (lane >= off) incl += t;
            }
            const int excl = incl - cnt;
            const bool has = e >= excl && e < incl;
            const unsigned long long holder = __ballot(has);
            if (holder == 0ull) return;  // fewer experts with pairs than slots (the same answer in all four wavefronts)
            uint32_t t = bits;
            for (int i = has ? e - excl : 0; i > 0; --i) t &= t - 1;
            const int mine = lane * 32 + (t ? __builtin_ctz(t) : 0);
            e = __shfl(mine, __builtin_ctzll(holder), 64);
        }
    }
    if constexpr (!PAIRS && !EARLY) {
        if (a.gl_slots > 0) {  // few rows over many experts: the workgroup's place is a slot, not an expert
            e = nth_expert_with_rows(a.gl, a.gl_type, a.E, e, lane);
            if (e < 0) return;
        }
    }
    const int8_t* we = expert_weights(a, e);
    const int8_t* w0 = we + ((int64_t)nb0 * KB) * 1024 + lane * 16;
    const int8_t* w1 = we + ((int64_t)nb1 * KB) * 1024 + lane * 16;

    // The weight addresses depend only on the unit, so the first batch of weight tiles is requested
    // before the expert's row range is known: the group-list lookup hides behind the HBM latency.
    v4i a0[UN], a1[UN];
    auto load_weights = [&](int kb) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int k = kb + u;
            if (k < kb_end) {
                a0[u] = gload16_nt(w0 + (int64_t)k * 1024);
                a1[u] = gload16_nt(w1 + (int64_t)k * 1024);
            } else {
                a0[u] = (v4i){0, 0, 0, 0};
                a1[u] = (v4i){0, 0, 0, 0};
            }
        }
    };
    if constexpr (EARLY) load_weights(kb_begin);

    int64_t row0 = 0, row1 = 0;
    if constexpr (PAIRS) {
        const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
        bool mine[4];
        int cnt = 0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            mine[c] = pid[c] == e;
            cnt += __popcll(__ballot(mine[c]));
        }
        if (lane == 0) pcount[wave] = cnt;
        __syncthreads();
        int base = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            if (w < wave) base += pcount[w];
            row1 += pcount[w];
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const unsigned long long m = __ballot(mine[c]);
            if (mine[c]) plist[base + __popcll(m & below)] = (uint16_t)(wave * Q + c * 64 + lane);
            base += __popcll(m);
        }
        __syncthreads();
        if (row1 == 0) return;  // the whole workgroup: nobody chose this expert
    } else {
        expert_rows(a.gl, a.gl_type, e, lane, row0, row1);
        if (!expert_in_launch(a, row1 - row0)) return;  // another kernel of this operator call covers the expert
        if (row1 > a.R) row1 = a.R;
        if (row1 <= row0) return;
    }
    if constexpr (!EARLY) load_weights(kb_begin);

    const int tok = lane & 31;
    const int kh = lane >> 5;

    // The channel scales of the runs this wavefront finishes (all four quarters, or quarter `wave` when K is
    // split) are requested together and before the first store of the epilogue: a load placed behind a store
    // waits for it (the memory counter retires in order), one round trip per run.  With K split they are two
    // registers and are requested in front of the K loop; the unsplit form requests them when the K loop has
    // ended, two quarters at a time (all eight together cost a wavefront of occupancy).
    constexpr int NQ = (KSPLIT == 1) ? 2 : 1;  // quarters whose scales are held at a time
    v4f cs0[NQ], cs1[NQ];
    auto load_channel_scales = [&](int q_first) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            cs0[i] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
            cs1[i] = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (EPI != EPI_I32) {
                const float* cs = expert_scales(a, e);
                const int ch = quad_channel(KSPLIT == 1 ? q_first + i : wave, lane);
                cs0[i] = gload4f(cs + nb0 * 32 + ch);
                cs1[i] = gload4f(cs + nb1 * 32 + ch);
            }
        }
    };
    if constexpr (KSPLIT > 1) load_channel_scales(0);

    for (int64_t r0 = row0; r0 < row1; r0 += 32) {
        const bool valid = r0 + tok < row1;
        int64_t row, src;  // where the row's result goes, where its values lie
        if constexpr (PAIRS) {
            row = plist[valid ? r0 + tok : 0];
            src = a.pair_gather ? row / a.pair_k : row;
        } else {
            row = r0 + tok;
            src = a.row_src ? (int64_t)a.row_src[valid ? row : row0] : row;
        }
        const int8_t* xr;
        float rs = 0.0f;
        if constexpr (!REQ) xr = a.x + src * a.K + kh * 16;
        if constexpr (REQ) {
            // rows r0 .. r0 + 31 of the expert -> int8 in LDS, every (row, four values) item by some thread
            const int pitch = a.K + 16;  // rows 16 bytes apart in the banks
            const int rows_now = (int)(row1 - r0 < 32 ? row1 - r0 : 32);
            const int per_row = a.K >> 2, items = rows_now * per_row;
            if (threadIdx.x < 32) qmax[threadIdx.x] = 0u;
            __syncthreads();
            for (int it = threadIdx.x; it < items; it += 256) {
                const int rr = it / per_row, c4 = it - rr * per_row;
                const v4f v = *(const v4f*)(a.y_in + (int64_t)plist[r0 + rr] * a.K + c4 * 4);
                float m = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float ab = __builtin_fabsf(v[j]);
                    m = ab > m ? ab : m;
                }
                atomicMax(&qmax[rr], __float_as_uint(m));
            }
            __syncthreads();
            for (int it = threadIdx.x; it < items; it += 256) {
                const int rr = it / per_row, c4 = it - rr * per_row;
                const v4f v = *(const v4f*)(a.y_in + (int64_t)plist[r0 + rr] * a.K + c4 * 4);
                const float amax = __uint_as_float(qmax[rr]);
                const float inv = 1.0f / (amax / 127.0f);
                uint32_t pk = 0u;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int8_t q = (amax == 0.0f) ? (int8_t)0 : sat_rint_i8(v[j] * inv);
                    pk |= (uint32_t)(uint8_t)q << (8 * j);
                }
                *(uint32_t*)(qtile + rr * pitch + c4 * 4) = pk;
            }
            if (threadIdx.x < rows_now) {
                const float amax = __uint_as_float(qmax[threadIdx.x]);
                qscale[threadIdx.x] = (amax == 0.0f) ? 0.0f : amax / 127.0f;
            }
            __syncthreads();
            xr = qtile + (valid ? tok : 0) * pitch + kh * 16;
            rs = qscale[valid ? tok : 0];
        } else if constexpr (EPI != EPI_I32) {
            rs = a.row_scale[(PAIRS || a.row_src) ? src : (valid ? row : row0)];
        }
        v16i c0 = {0}, c1 = {0};
        if (r0 != row0) load_weights(kb_begin);
        for (int kb = kb_begin; kb < kb_end; kb += UN) {
            v4i b[UN];
#pragma unroll
            for (int u = 0; u < UN; ++u)
                b[u] = (valid && kb + u < kb_end) ? *(const v4i*)(xr + (kb + u) * 32) : (v4i){0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < UN; ++u) {
                c0 = mfma_i8(a0[u], b[u], c0);
                c1 = mfma_i8(a1[u], b[u], c1);
            }
            if (kb + UN < kb_end) load_weights(kb + UN);
        }
        if constexpr (KSPLIT > 1) {
            // int32 partial sums of the four K slices meet in LDS (integer adds: exact, order free),
            // then every wavefront finishes one quarter of the channels
            if (wave == 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    red[v * 64 + lane] = c0[v];
                    red[(16 + v) * 64 + lane] = c1[v];
                }
            }
            __syncthreads();
            if (wave > 0) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    atomicAdd(&red[v * 64 + lane], c0[v]);
                    atomicAdd(&red[(16 + v) * 64 + lane], c1[v]);
                }
            }
            __syncthreads();
            int g[4], u[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                g[j] = red[(4 * wave + j) * 64 + lane];
                u[j] = red[(16 + 4 * wave + j) * 64 + lane];
            }
            const int ch = quad_channel(wave, lane);
            if constexpr (EPI == EPI_I32 && SLABS) {
                if (valid && a.acc_part) {
                    // the slab's partial sums to its own plane of the scratch; slab_sum_kernel adds the planes
                    int32_t* plane = a.acc_part + ((int64_t)blockIdx.y * a.R + row) * a.N;
                    *(v4i*)(plane + nb0 * 32 + ch) = (v4i){g[0], g[1], g[2], g[3]};
                    *(v4i*)(plane + nb1 * 32 + ch) = (v4i){u[0], u[1], u[2], u[3]};
                } else if (valid) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        atomicAdd(a.acc + row * a.N + nb0 * 32 + ch + j, g[j]);
                        atomicAdd(a.acc + row * a.N + nb1 * 32 + ch + j, u[j]);
                    }
                }
            } else {
                epilogue_run<EPI>(a, row, valid, nb0 * 32 + ch, nb1 * 32 + ch, g, u, rs, cs0[0], cs1[0]);
            }
            __syncthreads();
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (q % NQ == 0) load_channel_scales(q);  // two quarters per round trip
                int g[4] = {c0[4 * q], c0[4 * q + 1], c0[4 * q + 2], c0[4 * q + 3]};
                int u[4] = {c1[4 * q], c1[4 * q + 1], c1[4 * q + 2], c1[4 * q + 3]};
                const int ch = quad_channel(q, lane);
                epilogue_run<EPI>(a, row, valid, nb0 * 32 + ch, nb1 * 32 + ch, g, u, rs, cs0[q % NQ], cs1[q % NQ]);
            }
        }
    }
}

// ------------------------------------------------------------------ SwiGLU re-quantisation
// One wavefront per row: SwiGLU values y fp32 [R, I] -> row absmax -> int8 + scale.
// Rows at or beyond the last group are left untouched.
// NV > 0: the row (at most NV x 256 values) stays in registers between the two passes, so y is read once;
// NV == 0: any length, second pass re-reads the row.
template <int NV>
__global__ __launch_bounds__(256) void swiglu_requant_kernel(const float* __restrict__ y,
                                                             const int64_t* __restrict__ gl, int gl_type, int E,
                                                             int64_t R, int I, int8_t* __restrict__ q,
                                                             float* __restrict__ qs)
{
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= R) return;
    if (gl) {  // without a group list (pair order) every row is a row of some expert
        int64_t r0, total;
        expert_rows(gl, gl_type, E - 1, lane, r0, total);
        if (row >= total) return;
    }
    const v4f* yr = (const v4f*)(y + row * I);
    const int nvec = I >> 2;
    float amax = 0.0f;
    v4f held[NV > 0 ? NV : 1];
    if constexpr (NV > 0) {
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            const int i = lane + 64 * n;
            held[n] = i < nvec ? yr[i] : (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int n = 0; n < NV; ++n)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float ab = __builtin_fabsf(held[n][j]);
                amax = ab > amax ? ab : amax;
            }
    } else {
        for (int i = lane; i < nvec; i += 64) {
            const v4f v = yr[i];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float ab = __builtin_fabsf(v[j]);
                amax = ab > amax ? ab : amax;
            }
        }
    }
    amax = wave_max(amax);
    const float s = amax / 127.0f;
    const float inv = 1.0f / s;
    if (lane == 0) qs[row] = (amax == 0.0f) ? 0.0f : s;
    uint32_t* qr = (uint32_t*)(q + row * I);
    auto pack = [&](v4f v) {
        uint32_t pk = 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int8_t b = (amax == 0.0f) ? (int8_t)0 : sat_rint_i8(v[j] * inv);
            pk |= (uint32_t)(uint8_t)b << (8 * j);
        }
        return pk;
    };
    if constexpr (NV > 0) {
#pragma unroll
        for (int n = 0; n < NV; ++n) {
            const int i = lane + 64 * n;
            if (i < nvec) qr[i] = pack(held[n]);
        }
    } else {
        for (int i = lane; i < nvec; i += 64) qr[i] = pack(yr[i]);
    }
}

void launch_swiglu_requant(const float* y, const int64_t* gl, int gl_type, int E, int64_t R, int I, int8_t* q,
                           float* qs, hipStream_t st)
{
    const dim3 grid((unsigned)((R + 3) / 4));
#define MOE355_REQUANT(NV_) \
    hipLaunchKernelGGL(swiglu_requant_kernel<NV_>, grid, dim3(256), 0, st, y, gl, gl_type, E, R, I, q, qs)
    if (I <= 4 * 256) MOE355_REQUANT(4);
    else if (I <= 8 * 256) MOE355_REQUANT(8);
    else if (I <= 16 * 256) MOE355_REQUANT(16);
    else MOE355_REQUANT(0);
#undef MOE355_REQUANT
}

static int check_gmm(const void* x, const void* w, const int64_t* gl, int gl_type, int64_t rows, int64_t k, int64_t n,
                     int E)
{
    if (rows < 0 || k <= 0 || n <= 0 || E <= 0) return MOE355_E_ARG;
    if (gl_type != MOE355_GL_CUMSUM && gl_type != MOE355_GL_COUNT) return MOE355_E_ARG;
    if (n % 64 != 0 || k % 32 != 0) return MOE355_E_SHAPE;
    if (rows >= 0x7fffffffLL || n >= 0x7fffffffLL || k >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if ((int64_t)E * (n / 64) >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (rows > 0 && (!x || !w || !gl)) return MOE355_E_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return MOE355_E_SHAPE;
    return MOE355_OK;
}

// Measurement hook: events that bracket exactly the next grouped-GEMM kernel launched from
// this thread (set by moe355_profile_next_gemm, consumed by one launch).
static thread_local hipEvent_t t_ev_start = nullptr;
static thread_local hipEvent_t t_ev_stop = nullptr;

void take_profile_events(hipEvent_t& start, hipEvent_t& stop)
{
    start = t_ev_start;
    stop = t_ev_stop;
    t_ev_start = nullptr;
    t_ev_stop = nullptr;
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t* __restrict__ p, int64_t n4)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) ((v4i*)p)[i] = (v4i){0, 0, 0, 0};
}

// acc = sum of the slabs' planes, for the rows of the one expert (gl[0] of them: count and running sum are the
// same number for one expert); the other rows become zero.  Integer sums: exact in any order.
__global__ __launch_bounds__(256) void slab_sum_kernel(const int32_t* __restrict__ part, int slabs, int64_t R, int N,
                                                       const int64_t* __restrict__ gl, int32_t* __restrict__ acc)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // 16-byte piece of acc
    const int64_t n4 = R * (int64_t)N / 4;
    if (i >= n4) return;
    int64_t rows = gl[0];
    if (rows > R) rows = R;
    v4i s = {0, 0, 0, 0};
    if (i * 4 / N < rows) {
        for (int p = 0; p < slabs; ++p) {
            const v4i v = ((const v4i*)(part + (int64_t)p * R * N))[i];
            s = (v4i){s[0] + v[0], s[1] + v[1], s[2] + v[2], s[3] + v[3]};
        }
    }
    ((v4i*)acc)[i] = s;
}

template <typename KernelT>
static void launch_gemm(KernelT kernel, dim3 grid, hipStream_t st, const GmmArgs& a, hipEvent_t ev0, hipEvent_t ev1)
{
    if (ev0 || ev1) hipExtLaunchKernelGGL(kernel, grid, dim3(256), 0, st, ev0, ev1, 0, a);
    else hipLaunchKernelGGL(kernel, grid, dim3(256), 0, st, a);
}

// Rows per expert decide the kernel: few rows -> weight streaming over single wavefronts; many -> LDS-tiled
// MFMA kernel with 128-row tiles; in between, when K is long enough to amortise a tile's fill and epilogue, the
// weight-streaming tiles (up to 256 rows) that fetch an expert's weights once.  The host only knows the mean; the
// histogram may be skewed (real routers are), so next to the family chosen from the mean a second family covers
// the experts that fall outside its range, picked expert by expert on the device (GemmPlan below).
static int tiled_bm(const GmmArgs& a)
{
    if (a.K % 64 != 0) return 0;
#ifdef MOE355_DEV_KNOBS  // experiments only (never defined for the shipped library): force one kernel family
    static const char* force = getenv("MOE355_GEMM");
    if (force && force[0] == 's') return 0;
    if (force && force[0] == 't') return 128;
    if (force && force[0] == 'T') return 256;
    if (force && force[0] == 'u') return 64;
#endif
    const int64_t avg = a.R / a.E;
    if (avg < 48) {
        // Streaming wants every expert inside one 32-row pass.  Measured with uniform routing (the friendliest
        // case for it) at K = 7168 / 2048: 24 rows per expert on average 1407 / 84 us streaming against 1288 / 74 us
        // on the tiles, 32 rows 1957 / 115 against 1311 / 75, 16 rows 1223 / 73 against 1266 / 73, 8 rows 1119
        // against 1244; under Zipf(1.1) routing at 16 rows on average the tiles win as well (1260 against 1521).
        // Decode batches (fewer than 1024 rows) always stream.
        if (a.R < 1024 || avg < 12) return 0;
        // the list of 256-row tiles is built from 16-bit counters (tile_map_kernel, by_length)
        const bool wide_small = a.K >= 4096 && a.R / 256 + a.E < 32768;
        // 24..47 rows per expert: tiles.  With a long K the weight-streaming tiles (their one- and two-block forms
        // for the experts of up to 32 / 64 rows): uniform routing over 256 experts, K = 7168, 24 / 32 / 48 rows
        // 1255 / 1270 / 1286 us against 1283 / 1305 / 1322 us on the 128-row tiles (streaming 1373 / 1938 / 2706);
        // at K = 2048 the two kinds of tiles measure the same (664 / 677 / 697 against 664 / 680 / 703).
        if (avg >= 24) return wide_small ? 256 : 128;
        // 12..23 rows per expert: large products split the experts between both families (gemm_plan; streaming
        // alone leads the tiles up to 20 rows at K = 7168 and up to 24 at K = 2048: 612 against 654 us at 20); for
        // small ones the second launch costs more than it brings and the tiles alone are as fast as streaming
        return (int64_t)a.E * a.N * a.K >= (1ll << 30) ? 0 : 128;
    }
    // the list of 256-row tiles is built from 16-bit counters (tile_map_kernel, by_length)
    const bool wide_ok = a.R / 256 + a.E < 32768;
    if (avg <= 256 && a.K >= 4096 && wide_ok) return 256;
    // around 128 rows per expert most experts fit one wide tile of 128 or 160 rows and fetch their weights once,
    // which pays from K = 1024 on (measured: 6 % at K = 2048 and 1024, a loss at K = 768 and at 64 rows)
    if (avg >= 96 && avg <= 192 && a.K >= 1024 && wide_ok) return 256;
    return 128;
}

// What one operator call launches: the family chosen from the mean rows per expert, restricted to the experts it
// is good at, and (split > 0) the 128-row tiles for the experts above that range.
//   mean < 24 (12..23 for products of a GiB of weights and more, see tiled_bm; such products from one row per
//     expert on, smaller ones from 1024 rows on): streaming
//     for experts of at most 32 rows (one pass over their weights, and no request before the group list says that
//     the expert is theirs), tiles for the others -- a 500-row expert would otherwise stream its weights 16 times
//     while the units of the cold experts have long finished.  Measured at the DeepSeek-V3 shape with Zipf(1.1)
//     routing, 4096 rows: 1154 us against 1260 (tiles alone) and 1521 (streaming alone) over 244 touched experts;
//     533 against 568 and 1190 over the 90 touched experts of the benchmark's batch.
//   The weight-streaming tiles (mean 48..256) keep every expert: sending those above 256 rows to the 128-row
//     tiles measured the same on a Zipf(1.1) batch of 32,768 rows (2149 against 2180 us for the gate_up product,
//     1136 against 1119 us for the down product) and would cost the uniform batches an empty launch.
struct GemmPlan {
    int bm;        // 0 streaming, 64 / 128 LDS-tiled, 256 weight-streaming tiles
    int split;     // > 0: experts with more than `split` rows run on another family instead
    int split_bm;  // that family: 128 LDS-tiled, 256 weight-streaming tiles
};

static GemmPlan gemm_plan(const GmmArgs& a, bool have_tile_ws)
{
    GemmPlan p = {have_tile_ws ? tiled_bm(a) : 0, 0, 128};
    if (a.E == 1 && a.R <= 64) p.bm = 0;  // dense, few rows: the streaming kernel, one workgroup per 64 channels
    if (!have_tile_ws || a.K % 64 != 0 || a.E == 1) return p;
#ifdef MOE355_DEV_KNOBS
    static const char* force = getenv("MOE355_GEMM");
    if (force && force[0]) return p;
    static const char* sp = getenv("MOE355_SPLIT");  // "<rows>:<family>", e.g. 32:256
    if (sp && sp[0] && p.bm == 0 && a.R >= 1024) {  // experiments only
        p.split = atoi(sp);
        const char* c = strchr(sp, ':');
        p.split_bm = c ? atoi(c + 1) : 128;
        return p;
    }
#endif
    // a large product (a GiB of weights and more) over many experts with few rows on average.  Decode batches
    // too, from one row per expert on: on uniform routing the second launch finds nothing to do and costs 3 to 8 us,
    // on skewed routing the hot experts leave the streaming kernel (which also requests nothing for an idle expert
    // in this form).  DeepSeek-V3 shape through the sorted path, 32 / 64 / 112 tokens: uniform 1216 -> 1159,
    // 1500 -> 1490, 1648 -> 1656 us; Zipf(1.1) 529 -> 391, 640 -> 533, 796 -> 625 us.
    if (p.bm == 0 && a.R >= 128 && a.R >= (int64_t)a.E && (int64_t)a.E * a.N * a.K >= (1ll << 30)) {
        p.split = 32;
        // the experts above the border: weight-streaming tiles when K is long (an expert of up to 256 rows fetches
        // its weights once), 128-row tiles otherwise.  Measured on 512 tokens of Zipf(1.1) routing at the
        // DeepSeek-V3 shape: K = 7168 518 against 532 us for the pair of launches, K = 2048 the other way round
        // by as much; a border of 16 or 64 rows instead of 32 costs 70 / 40 us.
        if (a.K >= 4096 && a.R / 256 + a.E < 32768) p.split_bm = 256;
    }
    return p;
}

// One expert with enough rows and channels for the 256 x 256 tiles to fill the chip: the dense kernel (measured
// against the 128-row tiles: 13 to 17 % faster from 192 tiles on, 20 to 25 % slower at 64 to 128 tiles).
static bool dense_tiles(const GmmArgs& a)
{
    if (a.E != 1 || a.K % 64 != 0) return false;
#ifdef MOE355_DEV_KNOBS
    static const char* force = getenv("MOE355_GEMM");
    if (force && force[0] == 'D') return true;
    if (force && force[0]) return false;
#endif
    return ((a.R + 255) / 256) * ((int64_t)(a.N + 255) / 256) >= 192;
}

static size_t tiled_ws_max(int64_t rows, int E)
{
    // the smallest tile needs the longest tile list; a call that splits the experts over two families builds two
    return 2 * ((tiled_workspace_bytes(rows, E, 64) + 255) & ~(size_t)255);
}

// K slabs of the dense few-row product (one expert, at most 64 rows, a long K, too few pairs of tiles to fill
// the chip); 1 = not that case
static int dense_slabs(int64_t R, int K, int N, int E)
{
    const int64_t units = (int64_t)E * (N / 64);
    const int KB = K >> 5;
    if (E != 1 || R > 64 || units >= 256 || units < 1 || KB < 64) return 1;
    int slabs = (int)(512 / units);
    if (slabs > KB / 8) slabs = KB / 8;
    return slabs < 1 ? 1 : slabs;
}

template <int EPI>
static int launch_gemm_auto(const GmmArgs& a_in, void* tile_ws, hipStream_t st, void* part_ws = nullptr,
                            size_t part_bytes = 0)
{
    GmmArgs a = a_in;
    hipEvent_t ev0 = t_ev_start, ev1 = t_ev_stop;  // measurement hook: around the GEMM kernels of this call
    t_ev_start = nullptr;
    t_ev_stop = nullptr;
    if (dense_tiles(a)) {
        launch_dense(EPI, a, st, ev0, ev1);
        return launch_status();
    }
    const GemmPlan plan = gemm_plan(a, tile_ws != nullptr);
    // the second family's tile map lies behind the first one's
    void* tile_ws2 = tile_ws ? (char*)tile_ws + ((tiled_workspace_bytes(a.R, a.E, 64) + 255) & ~(size_t)255) : nullptr;
    if (plan.split > 0) a.rows_max = plan.split;
    hipEvent_t first_stop = plan.split > 0 ? nullptr : ev1;
    if (plan.bm) {
        launch_tiled_any(EPI, plan.bm, a, tile_ws, st, ev0, first_stop);
    } else {
        const int64_t units = (int64_t)a.E * (a.N / 64);
        bool done = false;
        if constexpr (EPI == EPI_I32) {
            // One expert with at most 64 rows (the shared expert of a decode batch: a dense product over a few
            // tokens): too few workgroups for a chip that needs thousands of loads in flight to stream at full rate.
            // K is cut into slabs, one workgroup per (pair of tiles, slab), partial sums added into the zeroed result.
            const int slabs = dense_slabs(a.R, a.K, a.N, a.E);
            if (slabs > 1) {
                const int64_t n4 = a.R * (int64_t)a.N / 4;  // N % 64 == 0
                const dim3 cover((unsigned)((n4 + 255) / 256));
                // with scratch for one plane per slab the partial sums are stored and added up afterwards;
                // without, they are added into the zeroed result with atomics (32 of 47 us at 8 slabs)
                const bool planes = part_ws && part_bytes >= (size_t)slabs * a.R * a.N * 4;
                if (planes) a.acc_part = (int32_t*)part_ws;
                else hipLaunchKernelGGL(zero_i32_kernel, cover, dim3(256), 0, st, a.acc, n4);
                launch_gemm(gmm_stream_kernel<EPI, 4, 4, 3, true>, dim3((unsigned)units, (unsigned)slabs), st, a, ev0,
                            first_stop);
                if (planes)
                    hipLaunchKernelGGL(slab_sum_kernel, cover, dim3(256), 0, st, a.acc_part, slabs, a.R, a.N, a.gl,
                                       a.acc);
                done = true;
            }
        }
        // Occupancy 3 keeps the SwiGLU epilogue out of scratch memory (131 registers).  With enough units to
        // fill the chip four times over and a short K, the down GEMM lets every wavefront stream a whole unit by
        // itself (no K split, no LDS reduction); otherwise the four wavefronts of a workgroup split K (from
        // K = 2048 on that measured 1.5 % faster on the whole layer, below it the same or slower).
        if (done) {
        } else if (plan.split == 0 && a.gl && a.R < (int64_t)a.E) {
            // fewer rows than experts (a decode batch of a few tokens on the sorted path): a slot per row instead
            // of a place per expert, so that the idle experts cost no dispatch; the workgroup looks up the expert
            // of its slot in the group list, so nothing is requested before that
            a.gl_slots = (int)a.R;
            launch_gemm(gmm_stream_kernel<EPI, 4, 4, 3, false, false>, dim3((unsigned)(a.R * (a.N / 64))), st, a, ev0,
                        first_stop);
        } else if (plan.split > 0) {
            launch_gemm(gmm_stream_kernel<EPI, 4, 4, 3, false, false>, dim3((unsigned)units), st, a, ev0, first_stop);
        } else if (EPI != EPI_SWIGLU && units >= 2048 && a.K < 2048) {
            launch_gemm(gmm_stream_kernel<EPI, 1, 4, 2>, dim3((unsigned)((units + 3) / 4)), st, a, ev0, first_stop);
        } else {
            launch_gemm(gmm_stream_kernel<EPI, 4, 4, 3>, dim3((unsigned)units), st, a, ev0, first_stop);
        }
    }
    if (plan.split > 0) {
        a.rows_min = plan.split + 1;
        a.rows_max = 0;
        launch_tiled_any(EPI, plan.split_bm, a, tile_ws2, st, nullptr, ev1);
    }
    return launch_status();
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe355_profile_next_gemm(void* start_event, void* stop_event)
{
    if ((start_event == nullptr) != (stop_event == nullptr)) return MOE355_E_ARG;
    t_ev_start = (hipEvent_t)start_event;
    t_ev_stop = (hipEvent_t)stop_event;
    return MOE355_OK;
}

extern "C" const char* moe355_gmm_kernel_name(int epilogue, int64_t rows, int64_t k, int64_t n, int num_experts)
{
    if (rows <= 0 || k <= 0 || n <= 0 || num_experts <= 0 || epilogue < 0 || epilogue > 2) return "";
    GmmArgs a = {};
    a.R = rows;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    if (dense_tiles(a)) return "gmm_dense_kernel";
    const GemmPlan p = gemm_plan(a, true);  // as launch_gemm_auto decides
    if (p.bm == 256) return "gmm_wide_kernel";
    if (p.bm != 0) return "gmm_tiled_kernel";
    if (!p.split) return "gmm_stream_kernel";
    return p.split_bm == 256 ? "gmm_stream_kernel + gmm_wide_kernel above 32 rows"
                             : "gmm_stream_kernel + gmm_tiled_kernel above 32 rows";
}

extern "C" int moe355_format_cast_nz(const int8_t* w, int layout, int64_t num_experts, int64_t n, int64_t k,
                                     int8_t* out, void* stream)
{
    if (num_experts <= 0 || n <= 0 || k <= 0 || !w || !out) return MOE355_E_ARG;
    if (layout != MOE355_W_ENK && layout != MOE355_W_EKN) return MOE355_E_ARG;
    if (n % 32 != 0 || k % 32 != 0) return MOE355_E_SHAPE;
    if (((uintptr_t)w & 15) || ((uintptr_t)out & 15)) return MOE355_E_SHAPE;
    const int64_t total = num_experts * n * k / 16;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipStream_t st = (hipStream_t)stream;
    if (layout == MOE355_W_ENK)
        hipLaunchKernelGGL(format_cast_nz_kernel<MOE355_W_ENK>, dim3((unsigned)blocks), dim3(256), 0, st, w,
                           num_experts, n, k, out);
    else
        hipLaunchKernelGGL(format_cast_nz_kernel<MOE355_W_EKN>, dim3((unsigned)blocks), dim3(256), 0, st, w,
                           num_experts, n, k, out);
    return launch_status();
}

extern "C" int moe355_gmm_i32(const int8_t* x, const int8_t* weight_nz, const int64_t* group_list,
                              int group_list_type, int64_t rows, int64_t k, int64_t n, int num_experts, int32_t* acc,
                              void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_gmm(x, weight_nz, group_list, group_list_type, rows, k, n, num_experts);
    if (rc != MOE355_OK) return rc;
    if (rows == 0) return MOE355_OK;
    if (!acc || ((uintptr_t)acc & 15)) return MOE355_E_ARG;
    // the scratch is optional here: without enough of it for the tile map the streaming kernel is used, and
    // what lies behind the tile map serves the partial sums of a product that cuts K into slabs
    const size_t map_bytes = (tiled_ws_max(rows, num_experts) + 255) & ~(size_t)255;
    void* tile_ws = (workspace && !((uintptr_t)workspace & 255) && workspace_bytes >= map_bytes) ? workspace : nullptr;
    void* part_ws = (tile_ws && workspace_bytes > map_bytes) ? (char*)workspace + map_bytes : nullptr;
    const size_t part_bytes = part_ws ? workspace_bytes - map_bytes : 0;
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.gl = group_list;
    a.gl_type = group_list_type;
    a.R = rows;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.acc = acc;
    return launch_gemm_auto<EPI_I32>(a, tile_ws, (hipStream_t)stream, part_ws, part_bytes);
}

extern "C" size_t moe355_gmm_i32_workspace(int64_t rows, int64_t n, int64_t k, int num_experts)
{
    if (rows <= 0 || n <= 0 || num_experts <= 0) return 256;
    size_t bytes = (tiled_ws_max(rows, num_experts) + 255) & ~(size_t)255;
    const int slabs = dense_slabs(rows, (int)k, (int)n, num_experts);
    if (slabs > 1) bytes += (size_t)slabs * rows * n * 4;  // one plane of partial sums per slab
    return bytes;
}

extern "C" size_t moe355_gmm1_swiglu_quant_workspace(int64_t rows, int64_t n, int64_t k, int num_experts)
{
    (void)k;
    (void)num_experts;
    if (rows <= 0 || n <= 0) return 256;
    return (((size_t)rows * (size_t)(n / 2) * 4 + 255) & ~(size_t)255) + tiled_ws_max(rows, num_experts);
}

static int gmm1_impl(const int8_t* x, const int8_t* weight_nz, const int8_t* const* weight_list,
                     const float* weight_scale, const float* const* scale_list, const float* x_scale,
                     const int64_t* group_list, int group_list_type, int64_t rows, int64_t k, int64_t n,
                     int num_experts, float swiglu_limit, int8_t* out, float* out_scale, void* workspace,
                     size_t workspace_bytes, void* stream, const int32_t* row_src = nullptr)
{
    const void* wany = weight_list ? (const void*)weight_list : (const void*)weight_nz;
    int rc = check_gmm(x, wany, group_list, group_list_type, rows, k, n, num_experts);
    if (rc != MOE355_OK) return rc;
    if (rows == 0) return MOE355_OK;
    if ((!weight_scale && !scale_list) || !x_scale || !out || !out_scale) return MOE355_E_ARG;
    if (((uintptr_t)weight_scale & 15) || ((uintptr_t)out & 3)) return MOE355_E_SHAPE;
    if (!workspace || ((uintptr_t)workspace & 255) ||
        workspace_bytes < moe355_gmm1_swiglu_quant_workspace(rows, n, k, num_experts))
        return MOE355_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    const int I = (int)(n / 2);
    float* y = (float*)workspace;
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.w_list = weight_list;
    a.gl = group_list;
    a.gl_type = group_list_type;
    a.R = rows;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.row_scale = x_scale;
    a.ch_scale = weight_scale;
    a.s_list = scale_list;
    a.limit = swiglu_limit;
    a.y = y;
    a.row_src = row_src;
    void* tile_ws = (char*)workspace + (((size_t)rows * I * 4 + 255) & ~(size_t)255);
    rc = launch_gemm_auto<EPI_SWIGLU>(a, tile_ws, st);
    if (rc != MOE355_OK) return rc;
    launch_swiglu_requant(y, group_list, group_list_type, num_experts, rows, I, out, out_scale, st);
    return launch_status();
}

extern "C" int moe355_gmm1_swiglu_quant(const int8_t* x, const int8_t* weight_nz, const float* weight_scale,
                                        const float* x_scale, const int64_t* group_list, int group_list_type,
                                        int64_t rows, int64_t k, int64_t n, int num_experts, float swiglu_limit,
                                        int8_t* out, float* out_scale, void* workspace, size_t workspace_bytes,
                                        void* stream)
{
    return gmm1_impl(x, weight_nz, nullptr, weight_scale, nullptr, x_scale, group_list, group_list_type, rows, k, n,
                     num_experts, swiglu_limit, out, out_scale, workspace, workspace_bytes, stream);
}

extern "C" int moe355_gmm1_swiglu_quant_gather(const int8_t* x, const float* x_scale, const int32_t* row_token,
                                               const int8_t* weight_nz, const float* weight_scale,
                                               const int64_t* group_list, int group_list_type, int64_t rows,
                                               int64_t k, int64_t n, int num_experts, float swiglu_limit, int8_t* out,
                                               float* out_scale, void* workspace, size_t workspace_bytes, void* stream)
{
    if (rows > 0 && !row_token) return MOE355_E_ARG;
    return gmm1_impl(x, weight_nz, nullptr, weight_scale, nullptr, x_scale, group_list, group_list_type, rows, k, n,
                     num_experts, swiglu_limit, out, out_scale, workspace, workspace_bytes, stream, row_token);
}

extern "C" int moe355_gmm1_swiglu_quant_list(const int8_t* x, const int8_t* const* weight_nz_list,
                                             const float* const* weight_scale_list, const float* x_scale,
                                             const int64_t* group_list, int group_list_type, int64_t rows, int64_t k,
                                             int64_t n, int num_experts, float swiglu_limit, int8_t* out,
                                             float* out_scale, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!weight_nz_list || !weight_scale_list) return MOE355_E_ARG;
    return gmm1_impl(x, nullptr, weight_nz_list, nullptr, weight_scale_list, x_scale, group_list, group_list_type,
                     rows, k, n, num_experts, swiglu_limit, out, out_scale, workspace, workspace_bytes, stream);
}

extern "C" size_t moe355_gmm2_dequant_workspace(int64_t rows, int64_t n, int64_t k, int num_experts)
{
    (void)n;
    (void)k;
    if (rows <= 0 || num_experts <= 0) return 256;
    return tiled_ws_max(rows, num_experts);
}

static int gmm2_impl(const int8_t* x, const int8_t* weight_nz, const int8_t* const* weight_list, const float* scale,
                     const float* const* scale_list, const float* per_token_scale, const int64_t* group_list,
                     int group_list_type, int64_t rows, int64_t k, int64_t n, int num_experts, void* out,
                     int out_dtype, void* workspace, size_t workspace_bytes, void* stream)
{
    const void* wany = weight_list ? (const void*)weight_list : (const void*)weight_nz;
    int rc = check_gmm(x, wany, group_list, group_list_type, rows, k, n, num_experts);
    if (rc != MOE355_OK) return rc;
    if (out_dtype != MOE355_DT_BF16 && out_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (rows > 0 && (!workspace || ((uintptr_t)workspace & 255) ||
                     workspace_bytes < moe355_gmm2_dequant_workspace(rows, n, k, num_experts)))
        return MOE355_E_WORKSPACE;
    if (rows == 0) return MOE355_OK;
    if ((!scale && !scale_list) || !per_token_scale || !out) return MOE355_E_ARG;
    if (((uintptr_t)scale & 15) || ((uintptr_t)out & 15)) return MOE355_E_SHAPE;
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.w_list = weight_list;
    a.gl = group_list;
    a.gl_type = group_list_type;
    a.R = rows;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.row_scale = per_token_scale;
    a.ch_scale = scale;
    a.s_list = scale_list;
    a.out = (uint16_t*)out;
    a.out_f16 = out_dtype == MOE355_DT_F16;
    return launch_gemm_auto<EPI_DEQUANT>(a, workspace, (hipStream_t)stream);
}

extern "C" int moe355_gmm2_dequant(const int8_t* x, const int8_t* weight_nz, const float* scale,
                                   const float* per_token_scale, const int64_t* group_list, int group_list_type,
                                   int64_t rows, int64_t k, int64_t n, int num_experts, void* out, int out_dtype,
                                   void* workspace, size_t workspace_bytes, void* stream)
{
    return gmm2_impl(x, weight_nz, nullptr, scale, nullptr, per_token_scale, group_list, group_list_type, rows, k, n,
                     num_experts, out, out_dtype, workspace, workspace_bytes, stream);
}

extern "C" int moe355_gmm2_dequant_list(const int8_t* x, const int8_t* const* weight_nz_list,
                                        const float* const* scale_list, const float* per_token_scale,
                                        const int64_t* group_list, int group_list_type, int64_t rows, int64_t k,
                                        int64_t n, int num_experts, void* out, int out_dtype, void* workspace,
                                        size_t workspace_bytes, void* stream)
{
    if (!weight_nz_list || !scale_list) return MOE355_E_ARG;
    return gmm2_impl(x, nullptr, weight_nz_list, nullptr, scale_list, per_token_scale, group_list, group_list_type,
                     rows, k, n, num_experts, out, out_dtype, workspace, workspace_bytes, stream);
}

// ------------------------------------------------------------------ pair order (decode batches)
extern "C" int moe355_gmm_pairs_supported(int64_t num_tokens, int top_k, int64_t n, int64_t k)
{
    return num_tokens > 0 && top_k > 0 && num_tokens * top_k <= kPairMax && n > 0 && k > 0 && n % 64 == 0 && k % 32 == 0;
}

// pair order: how many places the grid gets.  A place per expert lets a workgroup request its first weight tiles
// before it has seen a single id, which is the fastest form when nearly every expert has pairs -- and makes every
// idle expert cost the dispatch of its workgroups plus 32 KiB of weights requested for nothing.  A slot per pair
// (at most one per expert; the kernel looks up which expert a slot belongs to, and requests nothing before) costs
// every launch one exposed lookup, and nothing for idle experts.  Measured, whole layer under graph replay:
//   DeepSeek-V3 shape, uniform routing, 1 / 8 / 32 / 64 / 128 tokens: 307 -> 104, 567 -> 403, 1174 -> 1114,
//     1492 -> 1475, 1641 -> 1639 us; Zipf(1.1) routing, 96 / 128 tokens: 719 -> 599, 839 -> 731 us
//   Qwen3 shape, uniform, 1 / 4 / 16 / 64 / 128 tokens: 48 -> 38, 62 -> 42, 91 -> 86, 111.7 -> 114.3, 116 -> 120 us;
//     Zipf(1.1), 24 / 64 / 128 tokens: 80.5 -> 63.3, 108.9 -> 83.0, 169.6 -> 127.4 us
// The host cannot know the skew.  Slots wherever uniform routing loses nothing by them: up to two pairs per expert,
// and at any number of pairs when an expert has 48 units and more (the DeepSeek-V3 shape); with more pairs over
// experts of few units (the Qwen3 shape from 40 tokens on) a place per expert, which is the faster form on uniform
// routing and the slower one on skewed routing.  The bit map of the lookup holds 2048 experts.
static int pair_places(GmmArgs& a)
{
    const int64_t places = a.R < (int64_t)a.E ? a.R : (int64_t)a.E;
    const bool slots = a.R <= 2 * (int64_t)a.E || a.N / 64 >= 48;
    a.pair_slots = (slots && a.E <= 2048) ? (int)places : 0;
    return (int)(a.pair_slots > 0 ? places : a.E);
}

extern "C" size_t moe355_gmm1_swiglu_quant_pairs_workspace(int64_t num_tokens, int top_k, int64_t n)
{
    if (num_tokens <= 0 || top_k <= 0 || n <= 0) return 256;
    return (((size_t)num_tokens * top_k * (size_t)(n / 2) * 4 + 255) & ~(size_t)255);
}

extern "C" int moe355_gmm1_swiglu_quant_pairs(const int8_t* x, const float* x_scale, const int32_t* topk_ids,
                                              int64_t num_tokens, int top_k, const int8_t* weight_nz,
                                              const float* weight_scale, int64_t k, int64_t n, int num_experts,
                                              float swiglu_limit, int8_t* out, float* out_scale, void* workspace,
                                              size_t workspace_bytes, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || k <= 0 || n <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (num_tokens == 0) return MOE355_OK;
    if (!moe355_gmm_pairs_supported(num_tokens, top_k, n, k)) return MOE355_E_SHAPE;
    if ((int64_t)num_experts * (n / 64) >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (!x || !x_scale || !topk_ids || !weight_nz || !weight_scale || !out || !out_scale) return MOE355_E_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)weight_nz & 15) || ((uintptr_t)weight_scale & 15) || ((uintptr_t)out & 3))
        return MOE355_E_SHAPE;
    if (!workspace || ((uintptr_t)workspace & 255) ||
        workspace_bytes < moe355_gmm1_swiglu_quant_pairs_workspace(num_tokens, top_k, n))
        return MOE355_E_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    const int64_t rows = num_tokens * top_k;
    const int I = (int)(n / 2);
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.R = rows;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.row_scale = x_scale;
    a.ch_scale = weight_scale;
    a.limit = swiglu_limit;
    a.y = (float*)workspace;
    a.pair_ids = topk_ids;
    a.pair_k = top_k;
    a.pair_gather = 1;
    hipEvent_t ev0, ev1;
    take_profile_events(ev0, ev1);
    const int64_t units = (int64_t)pair_places(a) * (n / 64);
    launch_gemm(gmm_stream_kernel<EPI_SWIGLU, 4, 4, 3, false, true, true>, dim3((unsigned)units), st, a, ev0, ev1);
    launch_swiglu_requant(a.y, nullptr, 0, num_experts, rows, I, out, out_scale, st);
    return launch_status();
}

extern "C" int moe355_gmm2_dequant_pairs(const int8_t* x, const int8_t* weight_nz, const float* scale,
                                         const float* per_token_scale, const int32_t* topk_ids, int64_t num_tokens,
                                         int top_k, int64_t k, int64_t n, int num_experts, void* out, int out_dtype,
                                         void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || k <= 0 || n <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (out_dtype != MOE355_DT_BF16 && out_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (num_tokens == 0) return MOE355_OK;
    if (!moe355_gmm_pairs_supported(num_tokens, top_k, n, k)) return MOE355_E_SHAPE;
    if ((int64_t)num_experts * (n / 64) >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (!x || !weight_nz || !scale || !per_token_scale || !topk_ids || !out) return MOE355_E_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)weight_nz & 15) || ((uintptr_t)scale & 15) || ((uintptr_t)out & 15))
        return MOE355_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.R = num_tokens * top_k;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.row_scale = per_token_scale;
    a.ch_scale = scale;
    a.out = (uint16_t*)out;
    a.out_f16 = out_dtype == MOE355_DT_F16;
    a.pair_ids = topk_ids;
    a.pair_k = top_k;
    a.pair_gather = 0;
    hipEvent_t ev0, ev1;
    take_profile_events(ev0, ev1);
    const int64_t units = (int64_t)pair_places(a) * (n / 64);
    // as the sorted form chooses: a wavefront per unit when there are enough units and K is short, and the units
    // of an expert come in fours (a workgroup collects the pairs of one expert)
    if (units >= 2048 && k < 2048 && (n / 64) % 4 == 0)
        launch_gemm(gmm_stream_kernel<EPI_DEQUANT, 1, 4, 2, false, true, true>, dim3((unsigned)((units + 3) / 4)), st, a,
                    ev0, ev1);
    else
        launch_gemm(gmm_stream_kernel<EPI_DEQUANT, 4, 4, 3, false, true, true>, dim3((unsigned)units), st, a, ev0, ev1);
    return launch_status();
}

// gate_up GEMM + SwiGLU in pair order, the fp32 values left as they are (the down GEMM below re-quantises them)
extern "C" int moe355_gmm1_swiglu_pairs(const int8_t* x, const float* x_scale, const int32_t* topk_ids,
                                        int64_t num_tokens, int top_k, const int8_t* weight_nz,
                                        const float* weight_scale, int64_t k, int64_t n, int num_experts,
                                        float swiglu_limit, float* y, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || k <= 0 || n <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (num_tokens == 0) return MOE355_OK;
    if (!moe355_gmm_pairs_supported(num_tokens, top_k, n, k)) return MOE355_E_SHAPE;
    if ((int64_t)num_experts * (n / 64) >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (!x || !x_scale || !topk_ids || !weight_nz || !weight_scale || !y) return MOE355_E_ARG;
    if (((uintptr_t)x & 15) || ((uintptr_t)weight_nz & 15) || ((uintptr_t)weight_scale & 15) || ((uintptr_t)y & 15))
        return MOE355_E_SHAPE;
    GmmArgs a = {};
    a.x = x;
    a.w = weight_nz;
    a.R = num_tokens * top_k;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.row_scale = x_scale;
    a.ch_scale = weight_scale;
    a.limit = swiglu_limit;
    a.y = y;
    a.pair_ids = topk_ids;
    a.pair_k = top_k;
    a.pair_gather = 1;
    hipEvent_t ev0, ev1;
    take_profile_events(ev0, ev1);
    const int64_t units = (int64_t)pair_places(a) * (n / 64);
    launch_gemm(gmm_stream_kernel<EPI_SWIGLU, 4, 4, 3, false, true, true>, dim3((unsigned)units), (hipStream_t)stream, a,
                ev0, ev1);
    return launch_status();
}

// the form of the down GEMM that re-quantises: a wavefront per unit (many units, a short K) and 32 rows of K + 16
// bytes in LDS for each of the two workgroups of a compute unit
extern "C" int moe355_gmm2_requant_pairs_supported(int64_t num_tokens, int top_k, int64_t n, int64_t k, int num_experts)
{
    if (!moe355_gmm_pairs_supported(num_tokens, top_k, n, k) || num_experts <= 0) return 0;
    const int64_t units = (int64_t)num_experts * (n / 64);
    if (!(units >= 2048 && k < 2048 && (n / 64) % 4 == 0 && k % 4 == 0 && 32 * (k + 16) <= 48 * 1024)) return 0;
    // it pays up to about three rows per expert (measured on 128 experts of 2048 x 768: 24 / 32 / 48 tokens of eight
    // slots 98.4 / 102.8 / 109.7 us against 101.3 / 104.8 / 110.5 us with the launch of its own, 64 tokens 112.0
    // against 111.3, 128 tokens 119.6 against 115.8): every workgroup of an expert quantises all its rows again
    return num_tokens * top_k <= 3 * (int64_t)num_experts;
}

extern "C" int moe355_gmm2_requant_dequant_pairs(const float* y, const int8_t* weight_nz, const float* scale,
                                                 const int32_t* topk_ids, int64_t num_tokens, int top_k, int64_t k,
                                                 int64_t n, int num_experts, void* out, int out_dtype, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || k <= 0 || n <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (out_dtype != MOE355_DT_BF16 && out_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (num_tokens == 0) return MOE355_OK;
    if (!moe355_gmm2_requant_pairs_supported(num_tokens, top_k, n, k, num_experts)) return MOE355_E_SHAPE;
    if (!y || !weight_nz || !scale || !topk_ids || !out) return MOE355_E_ARG;
    if (((uintptr_t)y & 15) || ((uintptr_t)weight_nz & 15) || ((uintptr_t)scale & 15) || ((uintptr_t)out & 15))
        return MOE355_E_SHAPE;
    GmmArgs a = {};
    a.y_in = y;
    a.w = weight_nz;
    a.R = num_tokens * top_k;
    a.K = (int)k;
    a.N = (int)n;
    a.E = num_experts;
    a.ch_scale = scale;
    a.out = (uint16_t*)out;
    a.out_f16 = out_dtype == MOE355_DT_F16;
    a.pair_ids = topk_ids;
    a.pair_k = top_k;
    a.pair_gather = 0;
    hipEvent_t ev0, ev1;
    take_profile_events(ev0, ev1);
    const int64_t units = (int64_t)pair_places(a) * (n / 64);
    const unsigned lds = (unsigned)(32 * (k + 16));
    auto kernel = gmm_stream_kernel<EPI_DEQUANT, 1, 4, 2, false, true, true, true>;
    const dim3 grid((unsigned)((units + 3) / 4));
    if (ev0 || ev1) hipExtLaunchKernelGGL(kernel, grid, dim3(256), lds, (hipStream_t)stream, ev0, ev1, 0, a);
    else hipLaunchKernelGGL(kernel, grid, dim3(256), lds, (hipStream_t)stream, a);
    return launch_status();
}
