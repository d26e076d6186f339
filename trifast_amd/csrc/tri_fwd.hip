// Forward kernel instantiations and their launcher.
#include "tri_fwd.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct FwdFamily {
  static constexpr int kNumTiles = 8;
  // {NW, R, BK}: block of NW*32 queries x R pair rows, K/V streamed BK keys at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 queries x 1 row,  32 keys per stage (fits every dtype / head dim)
        {4, 2, 64},  // 1: 128 queries x 2 rows, 64 keys per stage
        {4, 4, 64},  // 2: 128 queries x 4 rows, 64 keys per stage
        {4, 4, 32},  // 3: 128 queries x 4 rows, 32 keys per stage
        {4, 2, 32},  // 4: 128 queries x 2 rows, 32 keys per stage (fewer registers: 3 waves per SIMD)
        {8, 4, 32},  // 5: 256 queries x 4 rows, 32 keys per stage
        {4, 2, 32 + kFwdFast},  // 6: tile 4 with the scheduled loop for workgroups without masked keys (16-bit types)
        {4, 4, 32 + kFwdFast},  // 7: tile 3 with the scheduled loop for workgroups without masked keys (16-bit types)
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int R, int BKF0>
  static hipError_t run(const FwdArgs& a, int bh, hipStream_t st, bool dry) {
    // (the scheduled loop exists for 16-bit types; elsewhere the tile is its general twin)
    constexpr int BK = BKF0 % kFwdFast;
    constexpr int BKF = (sizeof(T) == 2 && R >= 2 && D <= 64) ? BKF0 : BK;
    // two stages of: K and V rows of the R pair rows + one packed bias tile per wave and key tile
    // (or the three stages of the scheduled loop)
    constexpr int lds = fwd_main_lds_bytes(D, (int)sizeof(T), NW, R, BKF);
    // R rows of accumulators and Q operands per wave must stay in registers
    constexpr int acc_regs = R * (((D + 31) / 32) * 16 + D / 2 * (int)sizeof(T) / 4);
    if constexpr (lds <= kMaxLds && (acc_regs <= 160 || R == 1)) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * 32 - 1) / (NW * 32), ((a.N + R - 1) / R + 7) / 8 * 8, bh);
      const int lds_total = lds + KeyTileMasks::lds_bytes(a.nwords);  // + key-tile bitmaps
      if (lds_total > kMaxLds) return hipErrorInvalidConfiguration;
      return launch_dyn(tri_fwd_kernel<T, D, NW, R, BKF>, grid, dim3(NW * 64), lds_total, st, a);
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int fwd_num_tiles() { return FwdFamily::kNumTiles; }

TileInfo fwd_tile_info(int tile) {
  return TileInfo{FwdFamily::P(tile, 0) * 32, FwdFamily::P(tile, 2) % kFwdFast, FwdFamily::P(tile, 0)};
}

bool fwd_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= FwdFamily::kNumTiles || !head_dim_ok(d) || n < 1) return false;
  FwdArgs a{};
  return dispatch<FwdFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

hipError_t fwd_launch(const FwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<FwdFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
