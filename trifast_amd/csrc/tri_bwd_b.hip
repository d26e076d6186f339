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
  template <typename T, int D, int WJ, int WK>
  static constexpr int stage_bytes() {
    return (2 * 2 * WJ * 32 + 2 * 2 * WK * 32) * D * (int)sizeof(T) + 2 * (2 * WJ * 32) * 4 + 256;
  }
  template <typename T, int D, int WJ, int WK, int>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    // registers of one row's operands, the db accumulators and the bias tiles
    constexpr int frag_regs = (2 * WJ + 2 * WK) * (D / 2) * (int)sizeof(T) / 4;
    constexpr int stage = stage_bytes<T, D, WJ, WK>();
    constexpr int nbuf = 2 * stage <= kMaxLds ? 2 : 1;
    // the smallest tile always runs (at the price of register spills for large head dims)
    constexpr bool fits = stage <= kMaxLds && (2 * WJ * WK * 16 + frag_regs <= 320 || WJ * WK == 1);
    if constexpr (fits) {
      if (dry) return hipSuccess;
      const int lds = nbuf * stage;
      dim3 grid((a.N + 2 * WJ * 32 - 1) / (2 * WJ * 32), (a.N + 2 * WK * 32 - 1) / (2 * WK * 32), bh * a.nchunks);
      hipError_t e = launch_dyn(tri_bwd_b_kernel<T, D, WJ, WK, nbuf>, grid, dim3(256), lds, st, a);
      if (e != hipSuccess || a.nchunks == 1) return e;
      const int64_t count = (int64_t)bh * a.N * a.N;
      hipLaunchKernelGGL(tri_bwd_b_reduce_kernel<T>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st,
                         a.dbpart, reinterpret_cast<T*>(a.db), count, a.nchunks);
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

// The pair rows are split into chunks when one chunk would leave most of the
// GPU idle (few query/key blocks at small n); every tile uses the same split so
// that the workspace does not depend on the tile.
int bwd_b_chunks(int64_t n, int64_t bh) {
  const int64_t blocks = ((n + 127) / 128) * ((n + 127) / 128) * bh;
  int64_t chunks = (512 + blocks - 1) / blocks;
  const int64_t max_chunks = (n + 63) / 64;  // at least 64 rows per chunk
  if (chunks > max_chunks) chunks = max_chunks;
  if (chunks > 8) chunks = 8;
  if (chunks < 1) chunks = 1;
  return (int)chunks;
}

hipError_t bwd_b_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdBFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
