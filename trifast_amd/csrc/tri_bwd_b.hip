// db kernel instantiations and their launcher.
#include "tri_bwd_b.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdBFamily {
  static constexpr int kNumTiles = 3;
  // {WJ, WK, unused}: each wave owns WJ x WK tiles of 32 x 32; 2 x 2 waves per workgroup
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {2, 2, 0},  // 0: 128 queries x 128 keys per workgroup
        {1, 2, 0},  // 1:  64 queries x 128 keys
        {1, 1, 0},  // 2:  64 queries x  64 keys
    };
    return t[tile][which];
  }
  template <typename T, int D, int WJ, int WK, int>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    // registers of one row's operands; prefetching the next row doubles them
    constexpr int frag_regs = (2 * WJ + 2 * WK) * (D / 2) * (int)sizeof(T) / 4;
    constexpr bool prefetch = frag_regs <= 64;
    // one wave tile of db accumulators + bias must stay in registers
    constexpr bool fits = WJ * WK * 32 + (prefetch ? 2 : 1) * frag_regs <= 400;
    if constexpr (fits) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + 2 * WJ * 32 - 1) / (2 * WJ * 32), (a.N + 2 * WK * 32 - 1) / (2 * WK * 32), bh);
      hipLaunchKernelGGL((tri_bwd_b_kernel<T, D, WJ, WK, prefetch>), grid, dim3(256), 0, st, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int bwd_b_num_tiles() { return BwdBFamily::kNumTiles; }

TileInfo bwd_b_tile_info(int tile) {
  return TileInfo{2 * BwdBFamily::P(tile, 0) * 32, 2 * BwdBFamily::P(tile, 1) * 32, 4};
}

bool bwd_b_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= BwdBFamily::kNumTiles || !head_dim_ok(d) || n < 1) return false;
  BwdArgs a{};
  return dispatch<BwdBFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

hipError_t bwd_b_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdBFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
