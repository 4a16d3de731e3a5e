// Grouped int8 GEMM for many rows per expert (prefill): MFMA-bound, LDS-staged tokens.
//
// Workgroup tile: BM tokens x 256 channels, K consumed 64 at a time.  The four wavefronts own 64
// channels each (two 32-channel storage tiles: for the gate_up GEMM a gate tile and its up tile,
// so SwiGLU pairs meet in one lane).  Weights never touch LDS: a storage tile is one MFMA A
// operand and is loaded straight into registers, two iterations ahead.  Tokens are shared by the
// four wavefronts: global -> registers (three iterations ahead) -> LDS in MFMA-operand order
// (every B operand is one conflict-free 1 KiB ds_read_b128 sweep) -> MFMA.
// Tiles are enumerated (expert, row block) by a small map kernel from the group list; the 1-D
// grid is remapped so that all column blocks of a row block, and the row blocks of one expert,
// run on the same XCD (workgroup i goes to XCD i % 8) and share its L2.
#include <hip/hip_ext.h>

#include "gmm_common.h"
#include <type_traits>

#include "gmm_tiled.h"

namespace moe355 {

// One workgroup.  Thread t owns experts [t*seg, (t+1)*seg).  Tiles are numbered expert by expert.
// by_length (the 256-row weight-streaming tiles): the tiles are listed longest first -- 161..192 rows, 129..160,
// up to 128, then the tall ones (more than 192 rows, which become two shorter column items) -- so that the
// workgroups that start last are the short ones and the compute units finish closer together.
// rows_min / rows_max: experts whose row count lies outside [rows_min, rows_max] (rows_max 0: no upper bound) get
// no tiles (another kernel of the same operator call covers them); their rows still count for the offsets.
__global__ __launch_bounds__(256) void tile_map_kernel(const int64_t* __restrict__ gl, int gl_type, int E, int BM,
                                                       int max_tiles, TileMap tm, int by_length, int rows_min,
                                                       int rows_max)
{
    auto tiled_rows = [&](int64_t m) -> int64_t { return (m >= rows_min && (rows_max == 0 || m <= rows_max)) ? m : 0; };
    __shared__ int32_t part_rows[16];
    __shared__ int32_t part_tiles[16];
    if (by_length) {
        // class of a tile with m rows left in its expert; per-thread counts per class, two classes per scan
        auto cls = [](int64_t m) -> int { return m > 192 ? 3 : (m > 160 ? 0 : (m > 128 ? 1 : 2)); };
        const int tid = threadIdx.x;
        const int seg = (E + 255) / 256;
        const int e0 = tid * seg;
        auto rows_of = [&](int e) -> int64_t {
            int64_t m = (gl_type == MOE355_GL_COUNT) ? gl[e] : gl[e] - (e > 0 ? gl[e - 1] : 0);
            return m < 0 ? 0 : m;
        };
        int32_t rows = 0, n01 = 0, n23 = 0;  // counts packed 16 + 16 bits (at most max_tiles < 32768 tiles)
        for (int j = 0; j < seg; ++j) {
            const int e = e0 + j;
            if (e < E) {
                const int64_t m = rows_of(e);
                rows += (int32_t)m;
                for (int64_t r0 = 0; r0 < tiled_rows(m); r0 += BM) {
                    const int c = cls(m - r0);
                    if (c < 2) n01 += 1 << (16 * c);
                    else n23 += 1 << (16 * (c - 2));
                }
            }
        }
        int32_t all_rows, all01, all23;
        const int32_t rows_before = block_scan_exclusive_i32(rows, part_rows, all_rows);
        const int32_t b01 = block_scan_exclusive_i32(n01, part_tiles, all01);
        const int32_t b23 = block_scan_exclusive_i32(n23, part_tiles, all23);
        const int32_t total[4] = {all01 & 0xffff, all01 >> 16, all23 & 0xffff, all23 >> 16};
        const int32_t all_tiles = total[0] + total[1] + total[2] + total[3];
        if (tid == 0) tm.count[0] = all_tiles < max_tiles ? all_tiles : max_tiles;
        int32_t next[4] = {b01 & 0xffff, total[0] + (b01 >> 16), total[0] + total[1] + (b23 & 0xffff),
                           total[0] + total[1] + total[2] + (b23 >> 16)};
        int64_t row = rows_before;
        for (int j = 0; j < seg; ++j) {
            const int e = e0 + j;
            if (e < E) {
                const int64_t m = rows_of(e);
                for (int64_t r0 = 0; r0 < tiled_rows(m); r0 += BM) {
                    const int32_t t = next[cls(m - r0)]++;
                    if (t < max_tiles) {
                        tm.expert[t] = e;
                        tm.row_begin[t] = (int32_t)(row + r0);
                        tm.row_end[t] = (int32_t)(row + m);
                    }
                }
                row += m;
            }
        }
        return;
    }
    const int tid = threadIdx.x;
    const int seg = (E + 255) / 256;
    const int e0 = tid * seg;
    auto rows_of = [&](int e) -> int64_t {
        int64_t m = (gl_type == MOE355_GL_COUNT) ? gl[e] : gl[e] - (e > 0 ? gl[e - 1] : 0);
        return m < 0 ? 0 : m;
    };
    int32_t rows = 0, tiles = 0;
    for (int j = 0; j < seg; ++j) {
        const int e = e0 + j;
        if (e < E) {
            const int64_t m = rows_of(e);
            rows += (int32_t)m;
            tiles += (int32_t)((tiled_rows(m) + BM - 1) / BM);
        }
    }
    // exclusive prefix of rows and tiles over the threads (experts in order)
    int32_t all_rows, all_tiles;
    const int32_t rows_before = block_scan_exclusive_i32(rows, part_rows, all_rows);
    const int32_t tiles_before = block_scan_exclusive_i32(tiles, part_tiles, all_tiles);
    if (tid == 0) tm.count[0] = all_tiles < max_tiles ? all_tiles : max_tiles;
    int64_t row = rows_before;
    int32_t t = tiles_before;
    for (int j = 0; j < seg; ++j) {
        const int e = e0 + j;
        if (e < E) {
            const int64_t m = rows_of(e);
            for (int64_t r0 = row; r0 < row + tiled_rows(m); r0 += BM) {
                if (t < max_tiles) {
                    tm.expert[t] = e;
                    tm.row_begin[t] = (int32_t)r0;
                    tm.row_end[t] = (int32_t)(row + m);
                }
                ++t;
            }
            row += m;
        }
    }
}

constexpr int kBN = 256;  // channels per workgroup (4 wavefronts x 2 storage tiles)
constexpr int kBK = 64;   // K per pipeline stage (2 MFMA K steps)

// LDS of one workgroup: RING token stages of the tallest tile, reused by the epilogue patches
template <int EPI, int BMT, int RING>
struct TiledLds {
    static constexpr int BM = 32 * BMT;
    static constexpr int STAGE_BYTES = BM * kBK;               // tokens of one stage in LDS
    static constexpr int ROWB = 128 + 16;                      // epilogue patch: bytes per token row (padded)
    static constexpr int PATCHES = (EPI == EPI_I32) ? 2 : 1;   // 32-row patches per wavefront in the epilogue
    static constexpr int EPI_BYTES = 4 * PATCHES * 32 * ROWB;
    static constexpr int BYTES = RING * STAGE_BYTES > EPI_BYTES ? RING * STAGE_BYTES : EPI_BYTES;
};

// Epilogue of one wavefront: BMT token blocks x two 32-channel storage tiles (nb0, nb1) out of the MFMA
// accumulators.  In the accumulators a lane owns one token and scattered runs of four channels;
// written like that every store would touch 64 different cache lines.  The wavefront instead
// turns one 32-token block at a time through a private LDS patch (token-major, 128 data bytes per
// token and tile) and stores whole 128-byte row segments: 8 lanes per token row.
// FLAG, SwiGLU epilogue: the clamp is compiled in (as compares and selects it costs 8 of about 50 vector
// instructions per output, and the epilogue is bound by their number); dequant epilogue: the output is fp16
// instead of bf16.  The caller branches once.
template <int EPI, int BMT, bool FLAG>
__device__ __forceinline__ void tiled_epilogue_body(const GmmArgs& a, int e, v16i (&acc)[2][BMT], int64_t row0,
                                                    int64_t row_end, int nb0, int nb1, int8_t* patch, int lane)
{
    constexpr int ROWB = TiledLds<EPI, BMT, 3>::ROWB;
    const int tok = lane & 31;
    const int hi = lane >> 5;
    const float* cs = (a.ch_scale || a.s_list) ? expert_scales(a, e) : nullptr;
    v4f s0[4], s1[4];
    if constexpr (EPI != EPI_I32) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            s0[q] = gload4f(cs + nb0 * 32 + 8 * q + 4 * hi);
            s1[q] = gload4f(cs + nb1 * 32 + 8 * q + 4 * hi);
        }
    }
    // every token scale is requested before the first store: the memory counter retires in order, so a load
    // behind a block's stores would wait for their acknowledgement, once per token block
    float rs_all[BMT];
#pragma unroll
    for (int b = 0; b < BMT; ++b) {
        rs_all[b] = 0.0f;
        if constexpr (EPI != EPI_I32) {
            const int64_t row = row0 + b * 32 + tok;
            const int64_t rc = row < row_end ? row : row_end - 1;
            rs_all[b] = a.row_scale[a.row_src ? (int64_t)a.row_src[rc] : rc];
            if (row >= row_end) rs_all[b] = 0.0f;
        }
    }
    // ... and has arrived before it: the stores below sit behind "row < row_end" branches, and a wait for a
    // load that is still in flight at that point would have to assume that none of them was issued, which
    // turns it into a wait for every store of the block before
#pragma unroll
    for (int b = 0; b < BMT; ++b) asm volatile("" : "+v"(rs_all[b]));
#pragma unroll
    for (int b = 0; b < BMT; ++b) {
        const int64_t row = row0 + b * 32 + tok;
        const bool valid = row < row_end;
        const float rs = rs_all[b];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ch = 8 * q + 4 * hi;  // first of this lane's four channels inside the tile
            if constexpr (EPI == EPI_I32) {
                *(v4i*)(patch + tok * ROWB + ch * 4) =
                    (v4i){acc[0][b][4 * q], acc[0][b][4 * q + 1], acc[0][b][4 * q + 2], acc[0][b][4 * q + 3]};
                *(v4i*)(patch + 32 * ROWB + tok * ROWB + ch * 4) =
                    (v4i){acc[1][b][4 * q], acc[1][b][4 * q + 1], acc[1][b][4 * q + 2], acc[1][b][4 * q + 3]};
            } else if constexpr (EPI == EPI_DEQUANT) {
                v4u16 o0, o1;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    o0[j] = f32_to_half<FLAG ? MOE355_DT_F16 : MOE355_DT_BF16>(((float)acc[0][b][4 * q + j] * rs) * s0[q][j]);
                    o1[j] = f32_to_half<FLAG ? MOE355_DT_F16 : MOE355_DT_BF16>(((float)acc[1][b][4 * q + j] * rs) * s1[q][j]);
                }
                // both tiles are adjacent in the output row: 64 bf16 = 128 bytes per token
                *(v4u16*)(patch + tok * ROWB + ch * 2) = o0;
                *(v4u16*)(patch + tok * ROWB + 64 + ch * 2) = o1;
            } else {
                v4f yv;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float gg = ((float)acc[0][b][4 * q + j] * rs) * s0[q][j];
                    float uu = ((float)acc[1][b][4 * q + j] * rs) * s1[q][j];
                    if constexpr (FLAG) {
                        gg = gg > a.limit ? a.limit : gg;
                        uu = uu > a.limit ? a.limit : uu;
                        uu = uu < -a.limit ? -a.limit : uu;
                    }
                    yv[j] = m_silu(gg) * uu;
                }
                *(v4f*)(patch + tok * ROWB + ch * 4) = yv;
            }
        }
        // read back row-major: lane -> (row r8 + 8*p, 16-byte column c16)
        const int c16 = lane & 7, r8 = lane >> 3;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int r = r8 + 8 * p;
            const int64_t orow = row0 + b * 32 + r;
            if (orow < row_end) {
                if constexpr (EPI == EPI_I32) {
                    *(v4i*)(a.acc + orow * a.N + nb0 * 32 + c16 * 4) = *(const v4i*)(patch + r * ROWB + c16 * 16);
                    *(v4i*)(a.acc + orow * a.N + nb1 * 32 + c16 * 4) =
                        *(const v4i*)(patch + 32 * ROWB + r * ROWB + c16 * 16);
                } else if constexpr (EPI == EPI_DEQUANT) {
                    // Non-temporal stores for the two large outputs: written back through the L2 in the ordinary
                    // way they slowed the weight streams of every other workgroup (K loops 8 % longer).
                    __builtin_nontemporal_store(*(const v4i*)(patch + r * ROWB + c16 * 16),
                                                (v4i*)(a.out + orow * a.N + nb0 * 32 + c16 * 8));
                } else {
                    __builtin_nontemporal_store(*(const v4i*)(patch + r * ROWB + c16 * 16),
                                                (v4i*)(a.y + orow * (a.N >> 1) + nb0 * 32 + c16 * 4));
                }
            }
        }
    }
}

template <int EPI, int BMT>
__device__ __forceinline__ void tiled_epilogue(const GmmArgs& a, int e, v16i (&acc)[2][BMT], int64_t row0,
                                               int64_t row_end, int nb0, int nb1, int8_t* patch, int lane)
{
    if constexpr (EPI == EPI_SWIGLU) {
        if (a.limit > 0.0f) {
            tiled_epilogue_body<EPI, BMT, true>(a, e, acc, row0, row_end, nb0, nb1, patch, lane);
            return;
        }
    }
    if constexpr (EPI == EPI_DEQUANT) {
        if (a.out_f16) {
            tiled_epilogue_body<EPI, BMT, true>(a, e, acc, row0, row_end, nb0, nb1, patch, lane);
            return;
        }
    }
    tiled_epilogue_body<EPI, BMT, false>(a, e, acc, row0, row_end, nb0, nb1, patch, lane);
}

// One tile of BMT token blocks: rows [row0, row_end) of expert e (at most 32 * BMT of them are computed),
// column block nt.
// RING = depth of the operand ring in registers: weights are requested RING - 1 K blocks ahead, tokens RING.
// REM: K / 64 modulo RING when K / 64 >= RING (the closing steps are then specialised), -1 for any K.
template <int EPI, int BMT, int RING, int REM>  // BMT = token blocks of 32 per tile (BM = 32 * BMT)
__device__ __forceinline__ void tiled_body(const GmmArgs& a, int e, int64_t row0, int64_t row_end, int nt,
                                           int8_t* lds_raw)
{
    constexpr int STAGE_BYTES = TiledLds<EPI, BMT, RING>::STAGE_BYTES;
    constexpr int CHUNKS = STAGE_BYTES / 16 / 256;        // 16-byte chunks per thread per stage
    constexpr int ROWB = TiledLds<EPI, BMT, RING>::ROWB;
    constexpr int PATCHES = TiledLds<EPI, BMT, RING>::PATCHES;
    static_assert(CHUNKS >= 1, "a stage is at least one 16-byte chunk per thread");
    int8_t (*Bs)[STAGE_BYTES] = reinterpret_cast<int8_t (*)[STAGE_BYTES]>(lds_raw);

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;

    const int NB = a.N >> 5, KB = a.K >> 5;
    const int half_tiles = NB >> 1;
    // storage tiles of this wavefront
    int nb0, nb1;
    if constexpr (EPI == EPI_SWIGLU) {
        nb0 = nt * 4 + wave;          // gate tile
        nb1 = nb0 + half_tiles;       // its up tile
    } else {
        nb0 = nt * 8 + 2 * wave;
        nb1 = nb0 + 1;
    }
    const bool have = (EPI == EPI_SWIGLU) ? (nb0 < half_tiles) : (nb1 < NB);
    const int8_t* we = expert_weights(a, e);
    const int8_t* w0 = we + ((int64_t)(have ? nb0 : 0) * KB) * 1024 + lane * 16;
    const int8_t* w1 = we + ((int64_t)(have ? nb1 : 0) * KB) * 1024 + lane * 16;

    const int n_iter = a.K / kBK;

    v4i Areg[RING][2][2];   // [stage][tile][k step]
    v4i Breg[RING][CHUNKS];

    // Loads past the last K block or the last row are redirected to valid addresses instead of being
    // skipped (their results are never used): the loop body stays free of branches, so the compiler can
    // keep several stages of loads in flight with partial s_waitcnt counts.
    const int last_it = n_iter - 1;
    auto load_A = [&](int it, int st) {
        const int itc = it < last_it ? it : last_it;
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            Areg[st][0][s] = gload16(w0 + ((int64_t)itc * 2 + s) * 1024);
            Areg[st][1][s] = gload16(w1 + ((int64_t)itc * 2 + s) * 1024);
        }
    };
    const int8_t* xrow[CHUNKS];
    int lds_off[CHUNKS];
#pragma unroll
    for (int j = 0; j < CHUNKS; ++j) {
        // 16 consecutive lanes take 16 consecutive token rows at the same K chunk: their 16-byte LDS
        // writes then fall into 16 different bank groups (no conflicts), and a load instruction still
        // covers 16 rows x 64 contiguous bytes
        const int row = (tid & 15) + 16 * ((tid >> 6) + 4 * j);
        const int kc = (tid >> 4) & 3;
        int64_t r = row0 + row;
        if (r > row_end - 1) r = row_end - 1;  // rows past the expert's end duplicate its last row
        if (a.row_src) r = a.row_src[r];       // the row's values lie in the token's row
        xrow[j] = a.x + r * a.K + kc * 16;
        const int s = kc >> 1, kh = kc & 1;
        lds_off[j] = (((s * BMT + (row >> 5)) * 64) + kh * 32 + (row & 31)) * 16;
    }
    auto load_B = [&](int it, int st) {
        const int itc = it < last_it ? it : last_it;
#pragma unroll
        for (int j = 0; j < CHUNKS; ++j) Breg[st][j] = *(const v4i*)(xrow[j] + (int64_t)itc * kBK);
    };
    auto store_B = [&](int st) {
#pragma unroll
        for (int j = 0; j < CHUNKS; ++j) *(v4i*)(&Bs[st][lds_off[j]]) = Breg[st][j];
    };

    v16i acc[2][BMT];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int b = 0; b < BMT; ++b) acc[t][b] = (v16i){0};

    // B operands of one K step (BMT fragments of 1 KiB) live in registers; the two K steps of a stage
    // are double-buffered so that LDS reads of one step run under the MFMAs of the other.
    v4i bf0[BMT], bf1[BMT];
    auto read_frags = [&](v4i* dst, int st, int s) {
#pragma unroll
        for (int b = 0; b < BMT; ++b) dst[b] = *(const v4i*)(&Bs[st][((s * BMT + b) * 64 + lane) * 16]);
    };
    auto mma_step = [&](const v4i* frags, int st, int s) {
#pragma unroll
        for (int b = 0; b < BMT; ++b) {
            acc[0][b] = mfma_i8(Areg[st][0][s], frags[b], acc[0][b]);
            acc[1][b] = mfma_i8(Areg[st][1][s], frags[b], acc[1][b]);
        }
    };

    // ---- prologue.  After it the loads still in flight are, oldest first, A(0) B(1) A(1) B(2) ...: the same
    // order every iteration leaves behind, so the wait counts the compiler derives at the loop head are exact.
    // Every load of the prologue is requested before the first wait, so that the fill of the pipeline costs
    // one memory latency, not two.
    load_B(0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r + 1 < RING; ++r) {
        load_A(r, r);
        load_B(r + 1, r + 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    store_B(0);
    __syncthreads();
    read_frags(bf0, 0, 0);

    // One pipeline step on stage U (compile-time ring position) for K block I.  LA / LB: request the weights of
    // K block I + RING - 1 / the tokens of K block I + RING; SB: move the tokens of K block I + 1 to LDS.
#define MOE355_STEP(U, I, LA, LB, SB)                                                            \
    {                                                                                            \
        /* first K step: its MFMAs go first; the LDS traffic of the second K step and of the */  \
        /* next stage is issued in the gaps while the matrix pipe is busy                    */  \
        _Pragma("unroll") for (int b = 0; b < BMT; ++b)                                          \
        {                                                                                        \
            acc[0][b] = mfma_i8(Areg[(U)][0][0], bf0[b], acc[0][b]);                             \
            acc[1][b] = mfma_i8(Areg[(U)][1][0], bf0[b], acc[1][b]);                             \
            bf1[b] = *(const v4i*)(&Bs[(U)][((BMT + b) * 64 + lane) * 16]);                      \
            if ((SB) && b == 0) store_B(((U) + 1) % RING); /* B(I+1): registers -> LDS */        \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
        __syncthreads(); /* B(I+1) visible to all wavefronts */                                  \
        _Pragma("unroll") for (int b = 0; b < BMT; ++b)                                          \
        {                                                                                        \
            acc[0][b] = mfma_i8(Areg[(U)][0][1], bf1[b], acc[0][b]);                             \
            acc[1][b] = mfma_i8(Areg[(U)][1][1], bf1[b], acc[1][b]);                             \
            if (SB) bf0[b] = *(const v4i*)(&Bs[((U) + 1) % RING][(b * 64 + lane) * 16]);         \
            if ((LA) && b == 0) load_A((I) + RING - 1, ((U) + RING - 1) % RING);                 \
            if ((LB) && b == (BMT > 1 ? 1 : 0)) load_B((I) + RING, (U));                         \
            __builtin_amdgcn_sched_barrier(0);                                                   \
        }                                                                                        \
    }
    if constexpr (REM < 0) {
        // any K: whole passes through the ring run without any condition inside (exact wait counts), the remainder
        // is peeled; requests past the last K block are redirected to it (load_A, load_B)
        const int n_full = (n_iter / RING) * RING;
        for (int i0 = 0; i0 < n_full; i0 += RING) {
            MOE355_STEP(0, i0, 1, 1, 1)
            MOE355_STEP(1, i0 + 1, 1, 1, 1)
            MOE355_STEP(2, i0 + 2, 1, 1, 1)
        }
        if (n_iter - n_full >= 1) MOE355_STEP(0, n_full, 1, 1, 1)
        if (n_iter - n_full >= 2) MOE355_STEP(1, n_full + 1, 1, 1, 1)
    } else {
        // K / 64 = 3 q + REM with q >= 1 (the host picks the instantiation).  The last RING steps request nothing
        // that lies past the last K block (the weights of the last block are requested RING - 1 steps before it,
        // its tokens RING steps before); their ring positions follow from REM, so every step is written out with
        // its requests decided at compile time: no condition inside a step, exact waits, and a tile of 12 K blocks
        // issues 66 loads per wavefront instead of 80.
        static_assert(RING == 3, "the closing steps are written for a ring of three");
        const int n_pass = (n_iter - RING - REM) / RING;  // whole passes that request both operands
        int it = 0;
        for (int ps = 0; ps < n_pass; ++ps, it += RING) {
            MOE355_STEP(0, it, 1, 1, 1)
            MOE355_STEP(1, it + 1, 1, 1, 1)
            MOE355_STEP(2, it + 2, 1, 1, 1)
        }
        if constexpr (REM >= 1) MOE355_STEP(0, it, 1, 1, 1)
        if constexpr (REM >= 2) MOE355_STEP(1, it + 1, 1, 1, 1)
        it += REM;
        MOE355_STEP(REM % RING, it, 1, 0, 1)
        MOE355_STEP((REM + 1) % RING, it + 1, 0, 0, 1)
        MOE355_STEP((REM + 2) % RING, it + 2, 0, 0, 0)
    }
#undef MOE355_STEP

    __syncthreads();  // all wavefronts are done reading the token stages; LDS is reused below
    if (!have) return;
    tiled_epilogue<EPI, BMT>(a, e, acc, row0, row_end, nb0, nb1, lds_raw + wave * (PATCHES * 32 * ROWB), lane);
}

// The last tile of an expert is usually short.  Tiles of at most 64 rows run the two-block body (half the
// MFMAs and half the token traffic of a full tile) inside the same launch, next to the full tiles of their
// expert, so that they still find the expert's weights in the L2 of their XCD.
template <int EPI, int BMT, int RING, int REM>
__global__ __launch_bounds__(256, (BMT <= 2 ? 3 : 2)) void gmm_tiled_kernel(GmmArgs a, TileMap tm, int max_tiles, int n_col_blocks)
{
    __shared__ __attribute__((aligned(16))) int8_t lds_raw[TiledLds<EPI, BMT, RING>::BYTES];
    // ---- which tile: XCD-aware remap of the 1-D grid over the tiles that exist (workgroup i runs on
    // XCD i % 8; each XCD gets one contiguous eighth of the tile list, in order)
    const int total = tm.count[0] * n_col_blocks;
    const int per_xcd = (total + 7) / 8;
    const int slot = (int)(blockIdx.x / 8);
    const int item = (int)(blockIdx.x % 8) * per_xcd + slot;
    if (slot >= per_xcd || item >= total) return;
    const int mt = item / n_col_blocks;
    const int nt = item % n_col_blocks;
    const int e = tm.expert[mt];
    const int64_t row0 = tm.row_begin[mt];
    int64_t row_end = tm.row_end[mt];
    if (row_end > a.R) row_end = a.R;
    if (row0 >= row_end) return;
    if constexpr (BMT > 2) {
        if (row_end - row0 <= 64) {
            tiled_body<EPI, 2, RING, REM>(a, e, row0, row_end, nt, lds_raw);
            return;
        }
    }
    tiled_body<EPI, BMT, RING, REM>(a, e, row0, row_end, nt, lds_raw);
}

// ------------------------------------------------------------------ weight-streaming tiles
// Tiles for shapes whose grouped GEMM is bound by streaming the weights (a few hundred rows per expert at
// most).  A workgroup of eight wavefronts works on up to 256 rows of one expert, so that an expert with up to
// 256 rows fetches its weights from HBM exactly once; every wavefront computes its token blocks x one channel
// group (two storage tiles) with the accumulator layout and the epilogue of the 128-row tiles.
//   wide tile (at most 192 rows left): wavefront g = channel group g of 8, all 4, 5 or 6 token blocks of 32
//   -> 128 / 160 / 192 x 512;
//   tall tile (193..256 rows left): wavefront (h, g) = token half h x channel group g of 4 -> 256 x 256, twice
//   the token traffic per weight byte (tokens come from L2, and that traffic costs weight bandwidth).
// Both operands reach LDS by LDS-direct loads (no register staging, so the prefetch depth costs no registers),
// each into a ring of its own.  A weight stage holds the weights of 64 K values (every storage tile x 2 K steps
// is a contiguous 1 KiB MFMA operand that is copied as it lies), a token stage the tokens' 64 bytes (row-major,
// with a rotation of the 16-byte chunks).
// The compiler does not count LDS-direct loads against the LDS reads that consume them: the wait for a stage
// is written by hand, before the barrier that publishes the stage.
constexpr int kWideLdsBytes = 163840;

constexpr int ring_gcd(int a, int b) { return b == 0 ? a : ring_gcd(b, a % b); }

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

#define MOE355_GPTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define MOE355_LPTR(p) ((__attribute__((address_space(3))) void*)(p))

// NBLK: 32-row token blocks per wavefront (4 in a tall tile; 4, 5 or 6 in a wide one, so that an expert a little
// above 128 rows keeps the wide shape instead of paying the token traffic of a tall tile).
template <int EPI, bool WIDE, int NBLK = 4>
__device__ __forceinline__ void stream_tile_body(const GmmArgs& a, int e, int64_t row0, int64_t row_end, int nt,
                                                 int8_t* lds)
{
    static_assert(WIDE ? (NBLK >= 1 && NBLK <= 8) : NBLK == 4, "tall tiles have two halves of four blocks");
    constexpr int GROUPS = WIDE ? 8 : 4;            // channel groups (two storage tiles each) per workgroup
    constexpr int A_BYTES = GROUPS * 4096;          // weights of a stage
    constexpr int X_BYTES = WIDE ? NBLK * 2048 : 16384;  // tokens of a stage
    // Two rings.  The weights come from HBM: their ring takes the LDS that is left once the tokens (L2 hits,
    // a third of the latency) have a ring of at least three stages.  wide: 4 + 4 (4 + 3 with five token
    // blocks); tall: 6 + 4.
    constexpr int SX = WIDE ? (NBLK > 4 ? 3 : 4) : 4;
    constexpr int SW = (kWideLdsBytes - SX * X_BYTES) / A_BYTES;
    constexpr int XBASE = SW * A_BYTES;
    constexpr int CYCLE = SW / ring_gcd(SW, SX) * SX;  // steps after which both rings are back at stage 0
    constexpr int NA = WIDE ? 4 : 2;                // weight loads per wavefront and stage
    constexpr int ROWB = TiledLds<EPI, 4, 3>::ROWB;
    constexpr int PATCHES = TiledLds<EPI, 4, 3>::PATCHES;
    static_assert(8 * PATCHES * 32 * ROWB <= SW * A_BYTES + SX * X_BYTES, "epilogue patches fit the stages");
    static_assert(SW * A_BYTES + SX * X_BYTES <= kWideLdsBytes && SX >= 3 && SW >= SX, "stages fit LDS");
    static_assert(CYCLE % SW == 0 && CYCLE % SX == 0, "the unrolled steps return to stage 0 of both rings");

    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int h = WIDE ? 0 : wave >> 2;
    const int g = WIDE ? wave : wave & 3;
    const int NB = a.N >> 5, KB = a.K >> 5;
    const int half_tiles = NB >> 1;
    auto tiles_of = [&](int cg, int& t0, int& t1) -> bool {
        if constexpr (EPI == EPI_SWIGLU) {
            t0 = cg;
            t1 = cg + half_tiles;
            return cg < half_tiles;
        } else {
            t0 = 2 * cg;
            t1 = t0 + 1;
            return t1 < NB;
        }
    };
    // what this wavefront computes
    int nb0, nb1;
    const bool have = tiles_of(nt * GROUPS + g, nb0, nb1);
    const int64_t hrow0 = row0 + 128 * h;
    const bool active = have && hrow0 < row_end;

    // what this wavefront copies.  Weights: tall -- storage tile wave % 2 of group wave / 2; wide -- both
    // storage tiles of group wave; always both K steps of the stage (2 KiB contiguous per tile).
    const int8_t* we = expert_weights(a, e);
    const int8_t* wsrc[WIDE ? 2 : 1];
    if constexpr (WIDE) {
        wsrc[0] = we + (int64_t)(have ? nb0 : 0) * KB * 1024 + lane * 16;
        wsrc[1] = we + (int64_t)(have ? nb1 : 0) * KB * 1024 + lane * 16;
    } else {
        int l0, l1;
        const bool lhave = tiles_of(nt * GROUPS + (wave >> 1), l0, l1);
        wsrc[0] = we + (int64_t)(lhave ? ((wave & 1) ? l1 : l0) : 0) * KB * 1024 + lane * 16;
    }
    // Tokens: one load covers 16 rows x the 64 K bytes of a stage, four neighbouring lanes on one row (one
    // 64-byte line per lane quad).  LDS slot of (row r, 16-byte chunk c) inside its 16-row KiB:
    // 4 * (r % 16) + (c + (r % 16) / 4) % 4 -- the rotation spreads the MFMA operand reads (32 rows at one
    // chunk, 64 bytes apart) over all banks.  Wavefront w copies rows 32 w .. 32 w + 31 (tall: two loads) or
    // 16 w .. 16 w + 15 (wide); 16-row blocks that lie past the expert's last row are not loaded at all
    // (their products are never stored).
    // A wide tile of more than four blocks has more than eight 16-row pieces: wavefront w also copies piece
    // w + 8 when that exists.
    constexpr int XROWS = WIDE ? 16 : 32;
    constexpr int XSECOND = WIDE ? 8 * 16 : 16;     // rows between the first and the second piece of a wavefront
    constexpr bool X2 = !WIDE || NBLK > 4;
    const int xchunk = ((lane & 3) - (lane >> 4)) & 3;
    const int64_t xfirst = row0 + wave * XROWS;
    const bool x2 = X2 && (WIDE ? wave + 8 < 2 * NBLK : true) && xfirst + XSECOND < row_end;
    const int n_xloads = xfirst >= row_end ? 0 : (x2 ? 2 : 1);
    int64_t xr0 = xfirst + (lane >> 2), xr1 = xr0 + XSECOND;
    if (xr0 > row_end - 1) xr0 = row_end - 1;  // rows past the expert's end duplicate its last row
    if (xr1 > row_end - 1) xr1 = row_end - 1;
    if (a.row_src) {  // the rows' values lie in their tokens' rows
        xr0 = a.row_src[xr0];
        xr1 = a.row_src[xr1];
    }
    const int8_t* xsrc0 = a.x + xr0 * a.K + xchunk * 16;
    const int8_t* xsrc1 = a.x + xr1 * a.K + xchunk * 16;
    // operand reads of this lane: token l % 32 of a block, K half l / 32, K step s -> chunk 2 s + l / 32
    const int r16 = lane & 15;
    const int frag_off = XBASE + (h * 8 + ((lane >> 4) & 1)) * 1024 + r16 * 64;
    const int frag_s0 = frag_off + (((lane >> 5) + (r16 >> 2)) & 3) * 16;
    const int frag_s1 = frag_off + ((2 + (lane >> 5) + (r16 >> 2)) & 3) * 16;
    const int a_off = g * 4096 + lane * 16;

    const int n_iter = a.K / kBK;
    const int last_it = n_iter - 1;
    // loads past the last K block are redirected to it (never used), so that the number of loads in flight,
    // which the hand-written waits rely on, is the same in every step
    auto load_weights = [&](int it, int st) {
        const int itc = it < last_it ? it : last_it;
        int8_t* base = lds + st * A_BYTES;
        // plain cache policy: marked non-temporal, the same loads made the kernel 5 % slower
        if constexpr (WIDE) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int8_t* wp = wsrc[t] + (int64_t)itc * 2048;
                __builtin_amdgcn_global_load_lds(MOE355_GPTR(wp), MOE355_LPTR(base + wave * 4096 + t * 2048), 16, 0,
                                                 0);
                __builtin_amdgcn_global_load_lds(MOE355_GPTR(wp + 1024),
                                                 MOE355_LPTR(base + wave * 4096 + t * 2048 + 1024), 16, 0, 0);
            }
        } else {
            const int8_t* wp = wsrc[0] + (int64_t)itc * 2048;
            __builtin_amdgcn_global_load_lds(MOE355_GPTR(wp), MOE355_LPTR(base + wave * 2048), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(MOE355_GPTR(wp + 1024), MOE355_LPTR(base + wave * 2048 + 1024), 16, 0, 0);
        }
    };
    auto load_tokens = [&](int it, int st) {
        const int itc = it < last_it ? it : last_it;
        int8_t* base = lds + XBASE + st * X_BYTES;
        if (n_xloads >= 1)
            __builtin_amdgcn_global_load_lds(MOE355_GPTR(xsrc0 + (int64_t)itc * kBK),
                                             MOE355_LPTR(base + wave * (XROWS * 64)), 16, 0, 0);
        if constexpr (X2) {
            if (n_xloads >= 2)
                __builtin_amdgcn_global_load_lds(MOE355_GPTR(xsrc1 + (int64_t)itc * kBK),
                                                 MOE355_LPTR(base + (WIDE ? (wave + 8) * 1024 : wave * 2048 + 1024)),
                                                 16, 0, 0);
        }
    };

    v16i acc[2][NBLK];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int b = 0; b < NBLK; ++b) acc[t][b] = (v16i){0};

    // Every step requests the tokens SX - 1 steps ahead and then the weights SW - 1 steps ahead; the steps before
    // the first one do the same for what lies at or after K block 0, so that the order of the requests, which the
    // hand-written waits count on, is the same from the start.
#pragma unroll
    for (int j = 1 - SW; j < 0; ++j) {
        if (j + SX - 1 >= 0) load_tokens(j + SX - 1, j + SX - 1);
        load_weights(j + SW - 1, j + SW - 1);
    }

    // Requests that may still be in flight when the step d before the last one (d = kSteady: any step that is at
    // least SW - 1 before it) waits for the stage `ahead` steps after its own: everything requested behind that
    // stage's tokens.  The last SW - 1 steps request no weights and the last SX - 1 no tokens (nothing lies past the
    // last K block), so the counts shrink towards the end; each of those steps is compiled with its own.
    constexpr int kSteady = 1 << 20;
    auto in_flight = [](int d, int ahead, int nx) constexpr {
        int n = (SW > SX && d >= SW - SX + ahead) ? NA : 0;  // the weights requested right behind those tokens
        for (int m = 1; m <= SX - 2 - ahead; ++m) n += (d + m >= SX - 1 ? nx : 0) + (d + m >= SW - 1 ? NA : 0);
        return n;
    };
    // the steps d = SW - 2 .. 0 before the end (those that exist), each with its distance as a type
    auto closing_steps = [&](auto& step_fn, auto dfirst) {
        auto one = [&](auto self, auto dtag) -> void {
            constexpr int D = decltype(dtag)::value;
            if (D < n_iter) {
                const int it = last_it - D;
                step_fn(dtag, it % SW, it % SX, it);
            }
            if constexpr (D > 0) self(self, std::integral_constant<int, D - 1>{});
        };
        one(one, dfirst);
    };
    const int n_main = n_iter > SW - 1 ? n_iter - (SW - 1) : 0;  // steps that request both operands
    const int n_full = (n_main / CYCLE) * CYCLE;
    if constexpr (WIDE) {
        // One K block on stage uw of the weights and ux of the tokens.  Requests retire in order.  The younger of
        // the two requests that this step needs is its tokens (its weights, in the same step, if the rings are
        // equally deep): what was requested after it may still be in flight.  The barrier then covers the other
        // wavefronts and also says that everybody is done reading the stages that the next requests overwrite.
        auto step = [&](auto dtag, int uw, int ux, int it) {
            constexpr int D = decltype(dtag)::value;
            if (n_xloads == 2) wait_vmcnt<in_flight(D, 0, 2)>();
            else if (n_xloads == 1) wait_vmcnt<in_flight(D, 0, 1)>();
            else wait_vmcnt<in_flight(D, 0, 0)>();
            __builtin_amdgcn_s_barrier();
            if constexpr (D >= SX - 1) load_tokens(it + SX - 1, (ux + SX - 1) % SX);
            if constexpr (D >= SW - 1) load_weights(it + SW - 1, (uw + SW - 1) % SW);
            if (active) {
                const int8_t* wbase = lds + uw * A_BYTES;
                const int8_t* xbase = lds + ux * X_BYTES;
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const v4i a0 = *(const v4i*)(wbase + a_off + s * 1024);
                    const v4i a1 = *(const v4i*)(wbase + a_off + 2048 + s * 1024);
#pragma unroll
                    for (int b = 0; b < NBLK; ++b) {
                        const v4i f = *(const v4i*)(xbase + (s ? frag_s1 : frag_s0) + b * 2048);
                        acc[0][b] = mfma_i8(a0, f, acc[0][b]);
                        acc[1][b] = mfma_i8(a1, f, acc[1][b]);
                    }
                }
            }
        };
        constexpr std::integral_constant<int, kSteady> steady{};
        for (int i0 = 0; i0 < n_full; i0 += CYCLE) {
#pragma unroll
            for (int u = 0; u < CYCLE; ++u) step(steady, u % SW, u % SX, i0 + u);
        }
#pragma unroll
        for (int u = 0; u + 1 < CYCLE; ++u)
            if (n_full + u < n_main) step(steady, u % SW, u % SX, n_full + u);
        // the closing steps: ring positions known at run time only (three or four steps of a tile's dozens)
        closing_steps(step, std::integral_constant<int, SW - 2>{});
    } else {
        // Tall tiles are bound by the matrix units, and every wavefront meets the others at the barrier of every K
        // block: operand reads that start behind that barrier leave all eight wavefronts, both of each SIMD, without
        // an MFMA to issue until the first LDS answer is back.  So the operands stay one K step (32 values) ahead in
        // registers, across the barrier: a block waits for the stage AFTER its own (one stage less of prefetch
        // distance: the operands of a tall tile are L2 hits), runs its first K step on operands read during the block
        // before, reads the second K step's under those MFMAs and the next block's first under the second's.  Reads
        // and MFMAs are placed one by one (sched_barrier): an MFMA that waits for the matrix pipe holds up whatever
        // is queued behind it in the wavefront.
        v4i fa[2][2], fb[2][NBLK];  // [register set][tile] / [register set][token block]
        auto read_operands = [&](int set, int uw, int ux, int s, int part) {
            const int8_t* wbase = lds + uw * A_BYTES;
            const int8_t* xbase = lds + ux * X_BYTES;
            if (part == 0) {
                fa[set][0] = *(const v4i*)(wbase + a_off + s * 1024);
                fa[set][1] = *(const v4i*)(wbase + a_off + 2048 + s * 1024);
                fb[set][0] = *(const v4i*)(xbase + (s ? frag_s1 : frag_s0));
            } else {
                fb[set][part] = *(const v4i*)(xbase + (s ? frag_s1 : frag_s0) + part * 2048);
            }
        };
        // the stage of K block 0 has landed (for everybody): its first operands
        auto wait_stage = [&]() {
            // the younger request of the stage waited for is its tokens; behind them: the weights of that step and
            // every request of the later steps (the steps before the first have requested everything, redirected
            // to the last K block where a tile has fewer blocks than the rings are deep)
            if (n_xloads == 2) wait_vmcnt<in_flight(kSteady, 0, 2)>();
            else if (n_xloads == 1) wait_vmcnt<in_flight(kSteady, 0, 1)>();
            else wait_vmcnt<in_flight(kSteady, 0, 0)>();
        };
        auto wait_next_stage = [&](auto dtag) {
            constexpr int D = decltype(dtag)::value;
            if (n_xloads == 2) wait_vmcnt<in_flight(D, 1, 2)>();
            else if (n_xloads == 1) wait_vmcnt<in_flight(D, 1, 1)>();
            else wait_vmcnt<in_flight(D, 1, 0)>();
        };
        static_assert(SX >= 4, "a block reads the stage after its own: three stages in flight plus the one overwritten");
        wait_stage();
        __builtin_amdgcn_s_barrier();
        if (active) {
#pragma unroll
            for (int part = 0; part < NBLK; ++part) read_operands(0, 0, 0, 0, part);
        }
        auto step = [&](auto dtag, int uw, int ux, int it) {
            constexpr int D = decltype(dtag)::value;
            if constexpr (D > 0) wait_next_stage(dtag);  // stage it + 1 has landed
            __builtin_amdgcn_s_barrier();
            if constexpr (D >= SX - 1) load_tokens(it + SX - 1, (ux + SX - 1) % SX);
            if constexpr (D >= SW - 1) load_weights(it + SW - 1, (uw + SW - 1) % SW);
            if (active) {
                // K step 0 on set 0, reading K step 1 into set 1
#pragma unroll
                for (int b = 0; b < NBLK; ++b) {
                    acc[0][b] = mfma_i8(fa[0][0], fb[0][b], acc[0][b]);
                    acc[1][b] = mfma_i8(fa[0][1], fb[0][b], acc[1][b]);
                    read_operands(1, uw, ux, 1, b);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // K step 1 on set 1, reading the next block's K step 0 into set 0
#pragma unroll
                for (int b = 0; b < NBLK; ++b) {
                    acc[0][b] = mfma_i8(fa[1][0], fb[1][b], acc[0][b]);
                    acc[1][b] = mfma_i8(fa[1][1], fb[1][b], acc[1][b]);
                    if constexpr (D > 0) read_operands(0, (uw + 1) % SW, (ux + 1) % SX, 0, b);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        constexpr std::integral_constant<int, kSteady> steady{};
        for (int i0 = 0; i0 < n_full; i0 += CYCLE) {
#pragma unroll
            for (int u = 0; u < CYCLE; ++u) step(steady, u % SW, u % SX, i0 + u);
        }
#pragma unroll
        for (int u = 0; u + 1 < CYCLE; ++u)
            if (n_full + u < n_main) step(steady, u % SW, u % SX, n_full + u);
        closing_steps(step, std::integral_constant<int, SW - 2>{});
    }

    wait_vmcnt<0>();  // the redirected loads past the end still write LDS
    __builtin_amdgcn_s_barrier();
    if (!active) return;
    tiled_epilogue<EPI, NBLK>(a, e, acc, hrow0, row_end, nb0, nb1, lds + wave * (PATCHES * 32 * ROWB), lane);
}

template <int EPI>
__global__ __launch_bounds__(512, 1) void gmm_wide_kernel(GmmArgs a, TileMap tm, int max_tiles, int n_col_blocks,
                                                          int columns)
{
    extern __shared__ __attribute__((aligned(16))) int8_t wide_lds[];
    // Workgroup i runs on XCD i % 8.  The tiles (listed longest first) go round the XCDs, tile t to XCD t % 8, and
    // the `columns` workgroups of a tile (a column: 512 channels, two column blocks) follow each other on that XCD,
    // so they run at the same time and share the tile's tokens in its L2.  Nothing here depends on the number of
    // tiles: the tile's entries are requested together with the count they are checked against.
    const int slot = (int)(blockIdx.x / 8);
    const int mt = (slot / columns) * 8 + (int)(blockIdx.x % 8);
    const int col = slot % columns;
    if (mt >= max_tiles) return;
    const int count = tm.count[0];
    const int e = tm.expert[mt];
    const int64_t row0 = tm.row_begin[mt];
    int64_t row_end = tm.row_end[mt];
    if (mt >= count) return;
    if (row_end > a.R) row_end = a.R;
    if (row0 >= row_end) return;
    // An expert of a few rows (the cold ones of a skewed batch) runs the same body with one or two token blocks:
    // the matrix units draw their power whether a block's rows exist or not, and the kernel's clock follows it.
    if (row_end - row0 <= 32) {
        stream_tile_body<EPI, true, 1>(a, e, row0, row_end, col, wide_lds);
    } else if (row_end - row0 <= 64) {
        stream_tile_body<EPI, true, 2>(a, e, row0, row_end, col, wide_lds);
    } else if (row_end - row0 <= 128) {
        stream_tile_body<EPI, true>(a, e, row0, row_end, col, wide_lds);
    } else if (row_end - row0 <= 160) {
        stream_tile_body<EPI, true, 5>(a, e, row0, row_end, col, wide_lds);
    } else if (row_end - row0 <= 192) {
        stream_tile_body<EPI, true, 6>(a, e, row0, row_end, col, wide_lds);
    } else {
        // a tall tile is one column block wide: the column's two blocks one after the other
        stream_tile_body<EPI, false>(a, e, row0, row_end, 2 * col, wide_lds);
        if (2 * col + 1 < n_col_blocks) {
            __syncthreads();  // the first block's epilogue is out of LDS
            stream_tile_body<EPI, false>(a, e, row0, row_end, 2 * col + 1, wide_lds);
        }
    }
}

// One expert that owns every row (a dense product: the shared expert of a prefill batch): 256 x 256 tiles of the
// tall form, one workgroup per tile and compute unit, found by arithmetic on the expert's row count.  This shape
// is bound by the matrix units and, before them, by what the XCDs fetch: a tile reads 256 token rows and 256
// weight channels over the whole of K, and only tiles on the same XCD share those reads in its L2.  The 8 XCDs
// (workgroup i runs on XCD i % 8) therefore split the tile grid into xm x xn rectangles of pm x pn tiles, as
// square as the shape allows, instead of every XCD streaming all the weights.
template <int EPI>
__global__ __launch_bounds__(512, 1) void gmm_dense_kernel(GmmArgs a, int xn, int pm, int pn, int n_col_blocks)
{
    extern __shared__ __attribute__((aligned(16))) int8_t wide_lds[];
    const int xcd = (int)(blockIdx.x % 8);
    const int slot = (int)(blockIdx.x / 8);
    const int mt = (xcd / xn) * pm + slot / pn;
    const int nt = (xcd % xn) * pn + slot % pn;
    if (nt >= n_col_blocks) return;
    int64_t rows = a.gl[0];  // one group: its count and its running total are the same number
    if (rows > a.R) rows = a.R;
    const int64_t row0 = (int64_t)mt * 256;
    if (row0 >= rows) return;
    stream_tile_body<EPI, false>(a, 0, row0, rows, nt, wide_lds);
}

// ------------------------------------------------------------------ host side
size_t tiled_workspace_bytes(int64_t rows, int E, int BM)
{
    const int64_t max_tiles = rows / BM + E;
    return 256 + (size_t)(((max_tiles * 4 + 255) / 256) * 256) * 3;
}

template <int EPI, int BMT, int RING>
static void launch_tiled(const GmmArgs& a, void* workspace, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1)
{
    constexpr int BM = 32 * BMT;
    const int max_tiles = (int)(a.R / BM + a.E);
    const size_t arr = (size_t)(((size_t)max_tiles * 4 + 255) / 256) * 256;
    TileMap tm;
    tm.count = (int32_t*)workspace;
    tm.expert = (int32_t*)((char*)workspace + 256);
    tm.row_begin = (int32_t*)((char*)workspace + 256 + arr);
    tm.row_end = (int32_t*)((char*)workspace + 256 + 2 * arr);
    hipLaunchKernelGGL(tile_map_kernel, dim3(1), dim3(256), 0, st, a.gl, a.gl_type, a.E, BM, max_tiles, tm, 0, a.rows_min,
                       a.rows_max);
    const int channels = (EPI == EPI_SWIGLU) ? a.N / 2 : a.N;
    const int per_block = (EPI == EPI_SWIGLU) ? kBN / 2 : kBN;
    const int n_col_blocks = (channels + per_block - 1) / per_block;
    const int total = max_tiles * n_col_blocks;
    const int grid = ((total + 7) / 8) * 8;
    auto launch = [&](auto kernel) {
        if (ev0 || ev1)
            hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, st, ev0, ev1, 0, a, tm, max_tiles, n_col_blocks);
        else
            hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, st, a, tm, max_tiles, n_col_blocks);
    };
    // the closing steps of the K loop are compiled for K / 64 modulo the ring depth
    const int n_iter = a.K / kBK;
    if (n_iter < RING) launch(gmm_tiled_kernel<EPI, BMT, RING, -1>);
    else if (n_iter % RING == 0) launch(gmm_tiled_kernel<EPI, BMT, RING, 0>);
    else if (n_iter % RING == 1) launch(gmm_tiled_kernel<EPI, BMT, RING, 1>);
    else launch(gmm_tiled_kernel<EPI, BMT, RING, 2>);
}

template <int EPI>
static void launch_wide(const GmmArgs& a, void* workspace, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1)
{
    constexpr int BM = 256;
    constexpr int lds_bytes = kWideLdsBytes;
    static const hipError_t attr = hipFuncSetAttribute((const void*)gmm_wide_kernel<EPI>,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    (void)attr;
    const int max_tiles = (int)(a.R / BM + a.E);
    const size_t arr = (size_t)(((size_t)max_tiles * 4 + 255) / 256) * 256;
    TileMap tm;
    tm.count = (int32_t*)workspace;
    tm.expert = (int32_t*)((char*)workspace + 256);
    tm.row_begin = (int32_t*)((char*)workspace + 256 + arr);
    tm.row_end = (int32_t*)((char*)workspace + 256 + 2 * arr);
    hipLaunchKernelGGL(tile_map_kernel, dim3(1), dim3(256), 0, st, a.gl, a.gl_type, a.E, BM, max_tiles, tm, 1, a.rows_min,
                       a.rows_max);
    const int channels = (EPI == EPI_SWIGLU) ? a.N / 2 : a.N;
    const int per_block = (EPI == EPI_SWIGLU) ? kBN / 2 : kBN;
    const int n_col_blocks = (channels + per_block - 1) / per_block;
    const int columns = (n_col_blocks + 1) / 2;
    const int grid = 8 * ((max_tiles + 7) / 8) * columns;  // one workgroup per (tile, column), no idle ones
    if (ev0 || ev1)
        hipExtLaunchKernelGGL((gmm_wide_kernel<EPI>), dim3(grid), dim3(512), lds_bytes, st, ev0, ev1, 0, a, tm,
                              max_tiles, n_col_blocks, columns);
    else
        hipLaunchKernelGGL((gmm_wide_kernel<EPI>), dim3(grid), dim3(512), lds_bytes, st, a, tm, max_tiles,
                           n_col_blocks, columns);
}

template <int EPI>
static void launch_dense_t(const GmmArgs& a, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1)
{
    constexpr int lds_bytes = kWideLdsBytes;
    static const hipError_t attr = hipFuncSetAttribute((const void*)gmm_dense_kernel<EPI>,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    (void)attr;
    const int channels = (EPI == EPI_SWIGLU) ? a.N / 2 : a.N;
    const int per_block = (EPI == EPI_SWIGLU) ? kBN / 2 : kBN;
    const int n_col_blocks = (channels + per_block - 1) / per_block;
    const int row_tiles = (int)((a.R + 255) / 256);
    // the split of the 8 XCDs over rows x columns with the smallest rectangle perimeter (= bytes fetched per XCD)
    int xn = 1, best = 0;
    for (int c = 1; c <= 8; c *= 2) {
        const int per_m = (row_tiles + 8 / c - 1) / (8 / c), per_n = (n_col_blocks + c - 1) / c;
        const int cost = per_m + per_n;
        if (c == 1 || cost < best) {
            best = cost;
            xn = c;
        }
    }
    const int pm = (row_tiles + 8 / xn - 1) / (8 / xn), pn = (n_col_blocks + xn - 1) / xn;
    const int grid = 8 * pm * pn;
    if (ev0 || ev1)
        hipExtLaunchKernelGGL((gmm_dense_kernel<EPI>), dim3(grid), dim3(512), lds_bytes, st, ev0, ev1, 0, a, xn, pm, pn,
                              n_col_blocks);
    else
        hipLaunchKernelGGL((gmm_dense_kernel<EPI>), dim3(grid), dim3(512), lds_bytes, st, a, xn, pm, pn, n_col_blocks);
}

void launch_dense(int epi, const GmmArgs& a, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1)
{
    if (epi == EPI_I32) launch_dense_t<EPI_I32>(a, st, ev0, ev1);
    else if (epi == EPI_SWIGLU) launch_dense_t<EPI_SWIGLU>(a, st, ev0, ev1);
    else launch_dense_t<EPI_DEQUANT>(a, st, ev0, ev1);
}

void launch_tiled_any(int epi, int bm, const GmmArgs& a, void* workspace, hipStream_t st, hipEvent_t ev0,
                      hipEvent_t ev1)
{
#define MOE355_TILED(E_, B_) launch_tiled<E_, B_, 3>(a, workspace, st, ev0, ev1)
    if (bm == 256) {
        if (epi == EPI_I32) launch_wide<EPI_I32>(a, workspace, st, ev0, ev1);
        else if (epi == EPI_SWIGLU) launch_wide<EPI_SWIGLU>(a, workspace, st, ev0, ev1);
        else launch_wide<EPI_DEQUANT>(a, workspace, st, ev0, ev1);
    } else if (bm == 128) {
        if (epi == EPI_I32) MOE355_TILED(EPI_I32, 4);
        else if (epi == EPI_SWIGLU) MOE355_TILED(EPI_SWIGLU, 4);
        else MOE355_TILED(EPI_DEQUANT, 4);
    } else {
        if (epi == EPI_I32) MOE355_TILED(EPI_I32, 2);
        else if (epi == EPI_SWIGLU) MOE355_TILED(EPI_SWIGLU, 2);
        else MOE355_TILED(EPI_DEQUANT, 2);
    }
#undef MOE355_TILED
}

}  // namespace moe355
