// Forward kernel instantiations and their launcher.
#include "tri_fwd.hpp"
#include "tri_launch.hpp"

namespace tri {

namespace {
// {NW, QT, BK}; block_j = NW*QT*32
constexpr int kNumFwdTiles = 4;
constexpr int kFwdTiles[kNumFwdTiles][3] = {
    {4, 1, 32},   // 0: 128 queries x 32 keys
    {4, 2, 64},   // 1: 256 queries x 64 keys
    {2, 1, 32},   // 2:  64 queries x 32 keys (small n)
    {4, 1, 64},   // 3: 128 queries x 64 keys
};

template <typename T, int D, int NW, int QT, int BK>
constexpr bool lds_fits() {
  constexpr int PAD = 16 / sizeof(T);
  constexpr int DROWS = ((D + 31) / 32) * 32;
  return (BK * (D + PAD) + DROWS * (BK + PAD)) * sizeof(T) <= 64 * 1024;
}

template <typename T, int D, int NW, int QT, int BK>
hipError_t launch_one(const FwdArgs& a, int bh, hipStream_t st) {
  if constexpr (lds_fits<T, D, NW, QT, BK>()) {
    dim3 grid((a.N + NW * QT * 32 - 1) / (NW * QT * 32), a.N, bh);
    hipLaunchKernelGGL((tri_fwd_kernel<T, D, NW, QT, BK>), grid, dim3(NW * 64), 0, st, a);
    return hipGetLastError();
  } else {
    return hipErrorInvalidConfiguration;
  }
}

template <typename T, int D>
hipError_t launch_tile(const FwdArgs& a, int bh, int tile, hipStream_t st) {
  switch (tile) {
    case 0: return launch_one<T, D, 4, 1, 32>(a, bh, st);
    case 1: return launch_one<T, D, 4, 2, 64>(a, bh, st);
    case 2: return launch_one<T, D, 2, 1, 32>(a, bh, st);
    case 3: return launch_one<T, D, 4, 1, 64>(a, bh, st);
  }
  return hipErrorInvalidValue;
}

template <typename T>
hipError_t launch_d(const FwdArgs& a, int bh, int d, int tile, hipStream_t st) {
  switch (d) {
    case 16: return launch_tile<T, 16>(a, bh, tile, st);
    case 32: return launch_tile<T, 32>(a, bh, tile, st);
    case 64: return launch_tile<T, 64>(a, bh, tile, st);
    case 128: return launch_tile<T, 128>(a, bh, tile, st);
  }
  return hipErrorInvalidValue;
}
}  // namespace

int fwd_num_tiles() { return kNumFwdTiles; }

TileInfo fwd_tile_info(int tile) {
  return TileInfo{kFwdTiles[tile][0] * kFwdTiles[tile][1] * 32, kFwdTiles[tile][2], kFwdTiles[tile][0]};
}

bool fwd_supports(int tile, int64_t n, int d, int dtype) {
  if (tile < 0 || tile >= kNumFwdTiles || !head_dim_ok(d) || n < 1) return false;
  if (dtype == kF32 && d == 128 && kFwdTiles[tile][2] == 64) return false;  // LDS
  return true;
}

hipError_t fwd_launch(const FwdArgs& a, int bh, int d, int dtype, int tile, hipStream_t st) {
  switch (dtype) {
    case kF32: return launch_d<float>(a, bh, d, tile, st);
    case kBF16: return launch_d<__bf16>(a, bh, d, tile, st);
    case kF16: return launch_d<_Float16>(a, bh, d, tile, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace tri
