// Forward kernel instantiations and their launcher.
#include "tri_fwd.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct FwdFamily {
  static constexpr int kNumTiles = 7;
  // {NW, R, BK}: block of NW*32 queries x R pair rows, K/V streamed BK keys at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 queries x 1 row,  32 keys per stage (fits every dtype / head dim)
        {4, 2, 64},  // 1: 128 queries x 2 rows, 64 keys per stage
        {4, 4, 64},  // 2: 128 queries x 4 rows, 64 keys per stage
        {4, 4, 32},  // 3: 128 queries x 4 rows, 32 keys per stage
        {4, 2, 32},  // 4: 128 queries x 2 rows, 32 keys per stage (fewer registers: 3 waves per SIMD)
        {8, 4, 32},  // 5: 256 queries x 4 rows, 32 keys per stage
        {8, 2, 32},  // 6: 256 queries x 2 rows, 32 keys per stage
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int R, int BK>
  static hipError_t run(const FwdArgs& a, int bh, hipStream_t st, bool dry) {
    // two stages of: K and V rows of the R pair rows + one packed bias tile per wave and key tile
    constexpr int lds = 2 * ((2 * R * BK * D + NW * (BK / 32) * 1024) * (int)sizeof(T) + 256);
    // R rows of accumulators and Q operands per wave must stay in registers
    constexpr int acc_regs = R * (((D + 31) / 32) * 16 + D / 2 * (int)sizeof(T) / 4);
    if constexpr (lds <= kMaxLds && (acc_regs <= 160 || R == 1)) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * 32 - 1) / (NW * 32), ((a.N + R - 1) / R + 7) / 8 * 8, bh);
      const int lds_total = lds + KeyTileMasks::lds_bytes(a.nwords);  // + key-tile bitmaps
      if (lds_total > kMaxLds) return hipErrorInvalidConfiguration;
      return launch_dyn(tri_fwd_kernel<T, D, NW, R, BK>, grid, dim3(NW * 64), lds_total, st, a);
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int fwd_num_tiles() { return FwdFamily::kNumTiles; }

TileInfo fwd_tile_info(int tile) {
  return TileInfo{FwdFamily::P(tile, 0) * 32, FwdFamily::P(tile, 2), FwdFamily::P(tile, 0)};
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
