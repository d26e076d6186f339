// Instantiations of the row-resident backward kernel for one 16-bit element type
// (one translation unit per type, so that they compile in parallel).
#pragma once
#include "tri_bwd_row.hpp"
#include "tri_dispatch.hpp"

namespace tri {

// tile index -> key tiles per wave; a workgroup holds rows of up to 128 * KT keys
constexpr int kRowKT[kBwdRowTiles] = {2, 3, 4, 5, 6, 7, 8, 8};  // (the last one: several passes of 8)

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

// Rows of up to kRowMaxPasses * 1024 keys at head dim 32: one launch per 1024 keys (8 key
// tiles per wave), each complete for dk and dv of its keys and adding its part to dq; the
// last pass runs with as few key tiles per wave as hold what is left of the row.
constexpr int kRowMaxPasses = 8;
template <typename T, int D, int KT>
hipError_t bwd_row_pass(const BwdArgs& ap, int bh, hipStream_t st) {
  constexpr int lds = bwd_row_lds_bytes(D, (int)sizeof(T), KT, true);
  const int total = bh * ap.N;
  dim3 grid((unsigned)((total + 7) / 8 * 8));
  return launch_dyn(tri_bwd_row_kernel<T, D, KT, true>, grid, dim3(kRowWaves * 64), lds, st, ap);
}
template <typename T, int D>
hipError_t bwd_row_run_multi(const BwdArgs& a, int bh, hipStream_t st, bool dry) {
  if constexpr (D == 32) {
    constexpr int per_pass = kRowWaves * 8;  // key tiles of a full pass
    // (a row that one pass holds is the single-pass tile's)
    if (a.N <= per_pass * 32 || a.N > kRowMaxPasses * per_pass * 32) return hipErrorInvalidConfiguration;
    if (dry) return hipSuccess;
    if (!a.dq_lo) return hipErrorInvalidValue;
    const int passes = (a.nwords + per_pass - 1) / per_pass;
    for (int p = 0; p < passes; ++p) {
      BwdArgs ap = a;
      ap.key_tile0 = p * per_pass;
      ap.pass_flags = (p > 0 ? 1 : 0) | (p + 1 < passes ? 2 : 0);
      const int left = a.nwords - p * per_pass;  // key tiles from this pass on
      hipError_t e;
      switch ((left + kRowWaves - 1) / kRowWaves) {
        case 1:
        case 2: e = bwd_row_pass<T, D, 2>(ap, bh, st); break;
        case 3: e = bwd_row_pass<T, D, 3>(ap, bh, st); break;
        case 4: e = bwd_row_pass<T, D, 4>(ap, bh, st); break;
        case 5: e = bwd_row_pass<T, D, 5>(ap, bh, st); break;
        case 6: e = bwd_row_pass<T, D, 6>(ap, bh, st); break;
        default: e = bwd_row_pass<T, D, 8>(ap, bh, st); break;  // (7 key tiles per wave spill in this variant)
      }
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  } else {
    return hipErrorInvalidConfiguration;
  }
}

template <typename T, int D>
hipError_t bwd_row_dispatch_kt(const BwdArgs& a, int bh, int tile, hipStream_t st, bool dry) {
  switch (tile) {
#ifndef TRI_DEV_ONLY_BF16_D32
    case 0: return bwd_row_run<T, D, kRowKT[0]>(a, bh, st, dry);
    case 1: return bwd_row_run<T, D, kRowKT[1]>(a, bh, st, dry);
    case 2: return bwd_row_run<T, D, kRowKT[2]>(a, bh, st, dry);
    case 3: return bwd_row_run<T, D, kRowKT[3]>(a, bh, st, dry);
    case 4: return bwd_row_run<T, D, kRowKT[4]>(a, bh, st, dry);
    case 5: return bwd_row_run<T, D, kRowKT[5]>(a, bh, st, dry);
    case 7: return bwd_row_run_multi<T, D>(a, bh, st, dry);
#endif
    case 6: return bwd_row_run<T, D, kRowKT[6]>(a, bh, st, dry);
  }
  return hipErrorInvalidValue;
}

template <typename T>
hipError_t bwd_row_dispatch_d(const BwdArgs& a, int bh, int d, int tile, hipStream_t st, bool dry) {
  switch (d) {
#ifndef TRI_DEV_ONLY_BF16_D32  // (development builds: one instantiation compiles in seconds)
    case 16: return bwd_row_dispatch_kt<T, 16>(a, bh, tile, st, dry);
    case 64: return bwd_row_dispatch_kt<T, 64>(a, bh, tile, st, dry);
#endif
    case 32: return bwd_row_dispatch_kt<T, 32>(a, bh, tile, st, dry);
  }
  return hipErrorInvalidConfiguration;  // wider rows do not fit the register file
}

}  // namespace tri
