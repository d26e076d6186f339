// dk/dv kernel instantiations and their launcher.
#include "tri_bwd_kv.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdKVFamily {
  static constexpr int kNumTiles = 4;
  // {NW, R, BJ}: block of NW*32 keys x R pair rows, queries streamed BJ at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 64},  // 0: 128 keys x 1 row,  64 queries per stage (fits every dtype / head dim)
        {4, 2, 32},  // 1: 128 keys x 2 rows, 32 queries per stage
        {4, 2, 64},  // 2: 128 keys x 2 rows, 64 queries per stage
        {2, 2, 32},  // 3:  64 keys x 2 rows, 32 queries per stage
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int R, int BJ>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int stage = 2 * R * BJ * D * (int)sizeof(T) + 2 * R * BJ * 4 + NW * (BJ / 32) * 1024 * (int)sizeof(T);
    // K, V operands and the dk, dv accumulators of the R rows stay in registers
    constexpr int acc_regs = R * (2 * ((D + 31) / 32) * 16 + 2 * (D / 2) * (int)sizeof(T) / 4);
    // the one-row tile always runs (at the price of register spills for large head dims)
    constexpr int nbuf = 2 * stage <= kMaxLds ? 2 : 1;
    if constexpr (stage <= kMaxLds && (acc_regs <= 200 || R == 1)) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * 32 - 1) / (NW * 32), ((a.N + R - 1) / R + 7) / 8 * 8, bh);
      return launch_dyn(tri_bwd_kv_kernel<T, D, NW, R, BJ, nbuf>, grid, dim3(NW * 64), nbuf * stage, st, a);
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

// tile ids: the streaming tiles above, then the row-resident ones (tri_bwd_row.hpp)
constexpr int kRowKeyTiles[kBwdRowTiles] = {2, 3, 4, 5, 6, 7, 8, 64};  // (the last one: up to eight passes of 8)

hipError_t row_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st, bool dry) {
  switch (dtype) {
    case kBF16: return bwd_row_launch_bf16(a, bh, d, tile, st, dry);
    case kF16: return bwd_row_launch_f16(a, bh, d, tile, st, dry);
  }
  return hipErrorInvalidConfiguration;  // fp32 rows do not fit
}

}  // namespace

int bwd_kv_num_tiles() { return BwdKVFamily::kNumTiles + kBwdRowTiles; }

bool bwd_kv_tile_writes_dq(int tile) { return tile >= BwdKVFamily::kNumTiles && tile < bwd_kv_num_tiles(); }

TileInfo bwd_kv_tile_info(int tile) {
  // block_j = queries per LDS stage, block_k = keys per workgroup
  if (bwd_kv_tile_writes_dq(tile)) return TileInfo{32, 128 * kRowKeyTiles[tile - BwdKVFamily::kNumTiles], 4};
  return TileInfo{BwdKVFamily::P(tile, 2), BwdKVFamily::P(tile, 0) * 32, BwdKVFamily::P(tile, 0)};
}

bool bwd_kv_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= bwd_kv_num_tiles() || !head_dim_ok(d) || n < 1) return false;
  BwdArgs a{};
  a.N = (int)n;
  if (bwd_kv_tile_writes_dq(tile)) return row_launch(a, 1, d, dtype, tile - BwdKVFamily::kNumTiles, nullptr, true) == hipSuccess;
  return dispatch<BwdKVFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

hipError_t bwd_kv_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  if (bwd_kv_tile_writes_dq(tile)) return row_launch(a, bh, d, dtype, tile - BwdKVFamily::kNumTiles, st, false);
  return dispatch<BwdKVFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
