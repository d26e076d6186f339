// Forward kernel instantiations and their launcher.
#include "tri_fwd.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct FwdFamily {
  static constexpr int kNumTiles = 4;
  // {NW, QT, BK}: block of NW*QT*32 queries, K/V streamed BK keys at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 queries x 32 keys
        {4, 2, 64},  // 1: 256 queries x 64 keys
        {2, 1, 32},  // 2:  64 queries x 32 keys (small n)
        {4, 1, 64},  // 3: 128 queries x 64 keys
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int QT, int BK>
  static hipError_t run(const FwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int PAD = 16 / sizeof(T);
    constexpr bool fits = 2 * BK * (D + PAD) * sizeof(T) <= kMaxStaticLds;
    if constexpr (fits) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * QT * 32 - 1) / (NW * QT * 32), (a.N + 7) / 8 * 8, bh);
      hipLaunchKernelGGL((tri_fwd_kernel<T, D, NW, QT, BK>), grid, dim3(NW * 64), 0, st, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int fwd_num_tiles() { return FwdFamily::kNumTiles; }

TileInfo fwd_tile_info(int tile) {
  return TileInfo{FwdFamily::P(tile, 0) * FwdFamily::P(tile, 1) * 32, FwdFamily::P(tile, 2), FwdFamily::P(tile, 0)};
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
