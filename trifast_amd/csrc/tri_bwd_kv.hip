// dk/dv kernel instantiations and their launcher.
#include "tri_bwd_kv.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdKVFamily {
  static constexpr int kNumTiles = 4;
  // {NW, KT, BJ}: block of NW*KT*32 keys, queries streamed BJ at a time
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {4, 1, 32},  // 0: 128 keys x 32 queries
        {4, 1, 64},  // 1: 128 keys x 64 queries
        {4, 2, 64},  // 2: 256 keys x 64 queries
        {2, 1, 32},  // 3:  64 keys x 32 queries
    };
    return t[tile][which];
  }
  template <typename T, int D, int NW, int KT, int BJ>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int PAD = 16 / sizeof(T);
    constexpr int lds = 2 * BJ * (D + PAD) * (int)sizeof(T) + 8 * BJ;
    if constexpr (lds <= kMaxStaticLds) {
      if (dry) return hipSuccess;
      dim3 grid((a.N + NW * KT * 32 - 1) / (NW * KT * 32), (a.N + 7) / 8 * 8, bh);
      hipLaunchKernelGGL((tri_bwd_kv_kernel<T, D, NW, KT, BJ>), grid, dim3(NW * 64), 0, st, a);
      return hipGetLastError();
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int bwd_kv_num_tiles() { return BwdKVFamily::kNumTiles; }

TileInfo bwd_kv_tile_info(int tile) {
  // block_j = queries per LDS stage, block_k = keys per workgroup
  return TileInfo{BwdKVFamily::P(tile, 2), BwdKVFamily::P(tile, 0) * BwdKVFamily::P(tile, 1) * 32, BwdKVFamily::P(tile, 0)};
}

bool bwd_kv_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= BwdKVFamily::kNumTiles || !head_dim_ok(d) || n < 1) return false;
  BwdArgs a{};
  return dispatch<BwdKVFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

hipError_t bwd_kv_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdKVFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
