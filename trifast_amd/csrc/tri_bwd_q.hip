// dq (+ delta) kernel instantiations and their launcher.
#include "tri_bwd_q.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdQFamily {
  static constexpr int kNumTiles = 4;
  // {NW, QT, BK}
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 queries x 32 keys
        {4, 2, 64},  // 1: 256 queries x 64 keys
        {2, 1, 32},  // 2:  64 queries x 32 keys
        {4, 1, 64},  // 3: 128 queries x 64 keys
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int QT, int BK>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int PAD = 16 / sizeof(T);
    constexpr int lds = 2 * BK * (D + PAD) * (int)sizeof(T);
    if constexpr (lds <= kMaxStaticLds) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * QT * 32 - 1) / (NW * QT * 32), (a.N + 7) / 8 * 8, bh);
      hipLaunchKernelGGL((tri_bwd_q_kernel<T, D, NW, QT, BK>), grid, dim3(NW * 64), 0, st, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int bwd_q_num_tiles() { return BwdQFamily::kNumTiles; }

TileInfo bwd_q_tile_info(int tile) {
  return TileInfo{BwdQFamily::P(tile, 0) * BwdQFamily::P(tile, 1) * 32, BwdQFamily::P(tile, 2), BwdQFamily::P(tile, 0)};
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
