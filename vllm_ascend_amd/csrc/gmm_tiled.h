// Host interface of the LDS-tiled grouped GEMM (gmm_tiled.hip).
#pragma once

#include "gmm_common.h"

namespace moe355 {

// (expert, row block) tiles of one launch, built on the device from the group list.
struct TileMap {
    int32_t* count;      // [1]
    int32_t* expert;     // [max_tiles]
    int32_t* row_begin;  // [max_tiles]
    int32_t* row_end;    // [max_tiles] end of the expert's rows
};

// bytes of scratch for the tile map (BM = rows per tile: 64, 128 or 256)
size_t tiled_workspace_bytes(int64_t rows, int E, int BM);

// epi: EPI_*; bm: 64 or 128 (LDS-tiled kernel) or 256 (weight-streaming tiles).  ev0/ev1: optional events recorded around the GEMM kernel itself.
void launch_tiled_any(int epi, int bm, const GmmArgs& a, void* workspace, hipStream_t st, hipEvent_t ev0,
                      hipEvent_t ev1);

// One expert owning every row (a.E == 1): 256 x 256 tiles placed by arithmetic, no tile map, no scratch.
void launch_dense(int epi, const GmmArgs& a, hipStream_t st, hipEvent_t ev0, hipEvent_t ev1);

}  // namespace moe355
