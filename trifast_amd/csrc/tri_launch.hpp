// Launch-side declarations shared by the per-kernel translation units and the
// C ABI.  Each kernel family lives in its own .hip file so they build in parallel.
#pragma once
#include <hip/hip_runtime.h>
#include "tri_args.hpp"

namespace tri {

struct TileInfo { int block_j, block_k, num_waves; };

// dtype codes match include/trifast_hip.h
constexpr int kF32 = 0, kBF16 = 1, kF16 = 2;

int fwd_num_tiles();
TileInfo fwd_tile_info(int tile);
bool fwd_supports(int tile, int64_t n, int d, int dtype);
hipError_t fwd_launch(const FwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st);

int bwd_q_num_tiles();
TileInfo bwd_q_tile_info(int tile);
bool bwd_q_supports(int tile, int64_t n, int d, int dtype);
hipError_t bwd_q_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st);

int bwd_kv_num_tiles();
TileInfo bwd_kv_tile_info(int tile);
bool bwd_kv_supports(int tile, int64_t n, int d, int dtype);
hipError_t bwd_kv_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st);

// Row-resident tiles of the dk/dv family: they also produce dq (and the per-query
// planes the db kernel reads), so the dq kernel is not launched with them.  Their tile
// ids follow the streaming dk/dv tiles.
constexpr int kBwdRowTiles = 8;
bool bwd_kv_tile_writes_dq(int tile);
hipError_t bwd_row_launch_bf16(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry);
hipError_t bwd_row_launch_f16(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry);

int bwd_b_num_tiles();
TileInfo bwd_b_tile_info(int tile);
bool bwd_b_supports(int tile, int64_t n, int d, int dtype);
hipError_t bwd_b_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st);
int bwd_b_chunks(int64_t n, int64_t bh, int row_bytes);

hipError_t prep_launch(const MaskPrepArgs& m, int b, const BiasPrepArgs& a, int bh, int dtype, hipStream_t st);

inline bool head_dim_ok(int d) { return d == 16 || d == 32 || d == 64 || d == 128; }

}  // namespace tri
