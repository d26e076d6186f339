// Instantiations of the row-resident backward kernel for one 16-bit element type
// (one translation unit per type, so that they compile in parallel).
#pragma once
#include "tri_bwd_row.hpp"
#include "tri_dispatch.hpp"

namespace tri {

// tile index -> key tiles per wave; a workgroup holds rows of up to 128 * KT keys
constexpr int kRowKT[kBwdRowTiles] = {2, 4, 6, 8};

template <typename T, int D, int KT>
hipError_t bwd_row_run(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
  constexpr int DM = (D + 31) / 32;
  constexpr int lds = bwd_row_lds_bytes(D, (int)sizeof(T), KT);
  // the dk, dv accumulators of KT key tiles stay in registers (half of the file at most)
  if constexpr (2 * KT * DM * 16 <= 256 && lds <= kMaxLds) {
    if (a.N > kRowWaves * KT * 32) return hipErrorInvalidConfiguration;
    if (dry) return hipSuccess;
    const int total = bh * a.N;
    dim3 grid((unsigned)((total + 7) / 8 * 8));
    return launch_dyn(tri_bwd_row_kernel<T, D, KT>, grid, dim3(kRowWaves * 64), lds, st, a);
  } else {
    return hipErrorInvalidConfiguration;
  }
}

template <typename T, int D>
hipError_t bwd_row_dispatch_kt(const BwdArgs& a, int bh, int tile, hipStream_t st, bool dry) {
  switch (tile) {
    case 0: return bwd_row_run<T, D, kRowKT[0]>(a, bh, st, dry);
    case 1: return bwd_row_run<T, D, kRowKT[1]>(a, bh, st, dry);
    case 2: return bwd_row_run<T, D, kRowKT[2]>(a, bh, st, dry);
    case 3: return bwd_row_run<T, D, kRowKT[3]>(a, bh, st, dry);
  }
  return hipErrorInvalidValue;
}

template <typename T>
hipError_t bwd_row_dispatch_d(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry) {
  switch (d) {
    case 16: return bwd_row_dispatch_kt<T, 16>(a, bh, tile, st, dry);
    case 32: return bwd_row_dispatch_kt<T, 32>(a, bh, tile, st, dry);
    case 64: return bwd_row_dispatch_kt<T, 64>(a, bh, tile, st, dry);
  }
  return hipErrorInvalidConfiguration;  // wider rows do not fit the register file
}

}  // namespace tri
