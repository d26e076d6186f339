// db kernel instantiations and their launcher.
#include "tri_bwd_b.hpp"
#include "tri_dispatch.hpp"

namespace tri {
namespace {

struct BwdBFamily {
  static constexpr int kNumTiles = 5;
  // {WJ, WK, 16 * GJ + GK}: GJ x GK waves per workgroup, each owning WJ x WK tiles of 32 x 32
  static constexpr int P(int tile, int which) {
    constexpr int t[kNumTiles][3] = {
        {2, 2, 16 * 2 + 2},  // 0: 128 queries x 128 keys,  4 waves
        {1, 2, 16 * 2 + 2},  // 1:  64 queries x 128 keys,  4 waves
        {1, 1, 16 * 2 + 2},  // 2:  64 queries x  64 keys,  4 waves (fits every dtype / head dim)
        {1, 2, 16 * 4 + 2},  // 3: 128 queries x 128 keys,  8 waves
        {1, 1, 16 * 4 + 4},  // 4: 128 queries x 128 keys, 16 waves
    };
    return t[tile][which];
  }
  template <typename T, int D, int WJ, int WK, int G>
  static hipError_t run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
    constexpr int GJ = G / 16, GK = G % 16;
    constexpr int BJ = GJ * WJ * 32, BKB = GK * WK * 32;
    // registers of one row's operands, the db accumulators and the bias tiles
    constexpr int frag_regs = (2 * WJ + 2 * WK) * (D / 2) * (int)sizeof(T) / 4;
    constexpr int stage = bwd_b_stage_bytes(BJ, BKB, LdsTile<T, D>::ROWB);
    // ring of row buffers: up to 4 (loads run 3 rows ahead), as many as fit
    constexpr int nbuf = 4 * stage <= kMaxLds ? 4 : (3 * stage <= kMaxLds ? 3 : (2 * stage <= kMaxLds ? 2 : 1));
    // the smallest tile always runs (at the price of register spills for large head dims)
    constexpr bool fits = stage <= kMaxLds && (2 * WJ * WK * 16 + frag_regs <= 320 || (WJ * WK == 1 && GJ * GK == 4));
    if constexpr (fits) {
      if (dry) return hipSuccess;
      const int lds = nbuf * stage;
      const int groups = bh * a.nchunks;
      dim3 grid((a.N + BJ - 1) / BJ, (a.N + BKB - 1) / BKB, (groups + 7) / 8 * 8);
      hipError_t e = launch_dyn(tri_bwd_b_kernel<T, D, GJ, GK, WJ, WK, nbuf>, grid, dim3(GJ * GK * 64), lds, st, a);
      if (e != hipSuccess || a.nchunks == 1) return e;
      const int64_t count = (int64_t)bh * a.N * a.N;
      hipLaunchKernelGGL(tri_bwd_b_reduce_kernel<T>, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, a, count);
      return hipGetLastError();
    } else {
      return hipErrorInvalidConfiguration;
    }
  }
};

}  // namespace

int bwd_b_num_tiles() { return BwdBFamily::kNumTiles; }

TileInfo bwd_b_tile_info(int tile) {
  const int gj = BwdBFamily::P(tile, 2) / 16, gk = BwdBFamily::P(tile, 2) % 16;
  return TileInfo{gj * BwdBFamily::P(tile, 0) * 32, gk * BwdBFamily::P(tile, 1) * 32, gj * gk};
}

bool bwd_b_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= BwdBFamily::kNumTiles || !head_dim_ok(d) || n < 1) return false;
  BwdArgs a{};
  return dispatch<BwdBFamily>(a, 1, d, dtype, tile, nullptr, true) == hipSuccess;
}

// The pair rows are split into chunks when one chunk would leave part of the GPU idle;
// every tile uses the same split so that the workspace does not depend on the tile.
// The split follows a model of how the kernel occupies the GPU: the (batch*head, chunk)
// groups go to the 8 XCDs in turn (fewer than 8 groups share the XCDs between them, a whole
// number each), an XCD runs 32 workgroups of the large tiles at a time (one per CU), and a
// workgroup takes one unit per pair row plus a start-up of about 8: the time is
//   rounds of 32 workgroups on the fullest XCD  x  (rows per chunk + 8).
// Measured against it (h = 4, d = 32, 128 x 128 blocks, microseconds against units): n = 320,
// 5 chunks 73 / 72; 384, 6 chunks 79 / 72 and 8 chunks 115 / 112; 448, 4 chunks 120 / 120;
// 768, 2 chunks 776 / 784; 1024, 1 chunk 1040 / 1032.  Up to 8 chunks of at least 16 rows;
// with equal times the fewer chunks win (one chunk needs no partials and no reduce pass).
int bwd_b_chunks(int64_t n, int64_t bh, int row_bytes) {
  (void)row_bytes;
  const int64_t blocks = ((n + 127) / 128) * ((n + 127) / 128);  // per group
  const int64_t max_chunks = n / 16 < 1 ? 1 : (n / 16 > 8 ? 8 : n / 16);
  int64_t best = 1, best_cost = -1;
  for (int64_t c = 1; c <= max_chunks; ++c) {
    const int64_t groups = bh * c;
    // the groups are the grid's z extent (padded to a multiple of 8), at most 65535
    if (c > 1 && (groups + 7) / 8 * 8 > 65535) break;
    const int64_t on_xcd = groups >= 8 ? (groups + 7) / 8 * blocks : (blocks + 8 / groups - 1) / (8 / groups);
    const int64_t cost = (on_xcd + 31) / 32 * ((n + c - 1) / c + 8);
    if (best_cost < 0 || cost < best_cost) {
      best = c;
      best_cost = cost;
    }
  }
  return (int)best;
}

hipError_t bwd_b_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdBFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
