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

// The pair rows are split into chunks when one chunk would leave most of the
// GPU idle (few query/key blocks at small n); every tile uses the same split so
// that the workspace does not depend on the tile.
// (`row_bytes`: bytes of a row of q.  The default tile for 64-byte rows is one workgroup of
// 16 waves per CU, so 256 workgroups fill the GPU; the tiles of wider rows run two to four
// per CU.  Measured at n = 1024, h = 4, d = 32: one chunk instead of two, which needs no
// partials and no reduce pass, is 6 % faster.)
int bwd_b_chunks(int64_t n, int64_t bh, int row_bytes) {
  const int64_t blocks = ((n + 127) / 128) * ((n + 127) / 128) * bh;
  const int64_t target = row_bytes <= 64 ? 256 : 512;
  int64_t chunks = (target + blocks - 1) / blocks;
  const int64_t max_chunks = (n + 63) / 64;  // at least 64 rows per chunk
  if (chunks > max_chunks) chunks = max_chunks;
  if (chunks > 8) chunks = 8;
  if (chunks < 1) chunks = 1;
  // The kernel runs each (batch*head, chunk) group on one XCD: when the rows are split
  // anyway, make the number of groups a multiple of the 8 XCDs if the row count allows
  // it.  (One chunk stays one chunk: it needs no partials and no reduce pass.)
  if (chunks > 1) {
    int64_t g = bh % 8 == 0 ? 8 : (bh % 4 == 0 ? 4 : (bh % 2 == 0 ? 2 : 1));
    const int64_t m = 8 / g;  // chunks must be a multiple of m
    const int64_t rounded = (chunks + m - 1) / m * m;
    if (rounded <= max_chunks && rounded <= 8) chunks = rounded;
  }
  // the groups are the grid's z extent (padded to a multiple of 8), at most 65535
  while (chunks > 1 && (bh * chunks + 7) / 8 * 8 > 65535) --chunks;
  return (int)chunks;
}

hipError_t bwd_b_launch(const BwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  return dispatch<BwdBFamily>(a, bh, d, dtype, tile, st, false);
}

}  // namespace tri
