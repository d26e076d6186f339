// dq (+ delta) kernel instantiations and their launcher.
#include "tri_bwd_q.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdQFamily {
  static constexpr int kNumTiles = 4;
  // {NW, R, BK}: block of NW*32 queries x R pair rows, K/V streamed BK keys at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 queries x 1 row,  32 keys per stage (fits every dtype / head dim)
        {4, 2, 64},  // 1: 128 queries x 2 rows, 64 keys per stage
        {4, 2, 32},  // 2: 128 queries x 2 rows, 32 keys per stage
        {4, 4, 32},  // 3: 128 queries x 4 rows, 32 keys per stage
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int R, int BK>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int lds = 2 * ((2 * R * BK * D + NW * (BK / 32) * 1024) * (int)sizeof(T) + 256);
    // Q, dO operands and the dq accumulator of the R rows stay in registers
    constexpr int acc_regs = R * (((D + 31) / 32) * 16 + 2 * (D / 2) * (int)sizeof(T) / 4);
    if constexpr (lds <= kMaxLds && (acc_regs <= 160 || R == 1)) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * 32 - 1) / (NW * 32), ((a.N + R - 1) / R + 7) / 8 * 8, bh);
      const int lds_total = lds + KeyTileMasks::lds_bytes(a.nwords);  // + key-tile bitmaps
      if (lds_total > kMaxLds) return hipErrorInvalidConfiguration;
      return launch_dyn(tri_bwd_q_kernel<T, D, NW, R, BK>, grid, dim3(NW * 64), lds_total, st, a);
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int bwd_q_num_tiles() { return BwdQFamily::kNumTiles; }

TileInfo bwd_q_tile_info(int tile) {
  return TileInfo{BwdQFamily::P(tile, 0) * 32, BwdQFamily::P(tile, 2), BwdQFamily::P(tile, 0)};
}

bool bwd_q_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= BwdQFamily::kNumTiles || !head_dim_ok(d) || n < 1) return false;
  BwdArgs a{};
  return dispatch<BwdQFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

hipError_t bwd_q_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdQFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
