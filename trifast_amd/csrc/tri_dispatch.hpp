// Runtime (dtype, head dim, tile id) -> compile-time instantiation dispatch,
// shared by the four kernel families.  A family F provides
//   static constexpr int kNumTiles;                 (at most 8)
//   static constexpr int P(int tile, int which);    three ints per tile
//   template <typename T, int D, int A, int B, int C>
//   static hipError_t run(const Args&, int bh, hipStream_t, bool dry);
// run() returns hipErrorInvalidConfiguration when the instantiation does not fit
// the hardware (LDS), and launches nothing when dry is set.
#pragma once
#include <hip/hip_runtime.h>
#include "tri_launch.hpp"

namespace tri {

template <class F, typename T, int D, class Args>
hipError_t dispatch_tile(const Args& a, int bh, int tile, hipStream_t st, bool dry) {
  switch (tile) {
    case 0: return F::template run<T, D, F::P(0, 0), F::P(0, 1), F::P(0, 2)>(a, bh, st, dry);
    case 1: if constexpr (F::kNumTiles > 1) return F::template run<T, D, F::P(1, 0), F::P(1, 1), F::P(1, 2)>(a, bh, st, dry); break;
    case 2: if constexpr (F::kNumTiles > 2) return F::template run<T, D, F::P(2, 0), F::P(2, 1), F::P(2, 2)>(a, bh, st, dry); break;
    case 3: if constexpr (F::kNumTiles > 3) return F::template run<T, D, F::P(3, 0), F::P(3, 1), F::P(3, 2)>(a, bh, st, dry); break;
    case 4: if constexpr (F::kNumTiles > 4) return F::template run<T, D, F::P(4, 0), F::P(4, 1), F::P(4, 2)>(a, bh, st, dry); break;
    case 5: if constexpr (F::kNumTiles > 5) return F::template run<T, D, F::P(5, 0), F::P(5, 1), F::P(5, 2)>(a, bh, st, dry); break;
    case 6: if constexpr (F::kNumTiles > 6) return F::template run<T, D, F::P(6, 0), F::P(6, 1), F::P(6, 2)>(a, bh, st, dry); break;
    case 7: if constexpr (F::kNumTiles > 7) return F::template run<T, D, F::P(7, 0), F::P(7, 1), F::P(7, 2)>(a, bh, st, dry); break;
  }
  return hipErrorInvalidValue;
}

template <class F, typename T, class Args>
hipError_t dispatch_d(const Args& a, int bh, int d, int tile, hipStream_t st, bool dry) {
  switch (d) {
#ifndef TRI_DEV_ONLY_BF16_D32  // (development builds: one instantiation family compiles in seconds)
    case 16: return dispatch_tile<F, T, 16>(a, bh, tile, st, dry);
    case 64: return dispatch_tile<F, T, 64>(a, bh, tile, st, dry);
    case 128: return dispatch_tile<F, T, 128>(a, bh, tile, st, dry);
#endif
    case 32: return dispatch_tile<F, T, 32>(a, bh, tile, st, dry);
  }
  return hipErrorInvalidValue;
}

template <class F, class Args>
hipError_t dispatch(const Args& a, int bh, int d, int dtype, int tile, hipStream_t st, bool dry) {
  switch (dtype) {
#ifndef TRI_DEV_ONLY_BF16_D32
    case kF32: return dispatch_d<F, float>(a, bh, d, tile, st, dry);
    case kF16: return dispatch_d<F, _Float16>(a, bh, d, tile, st, dry);
#endif
    case kBF16: return dispatch_d<F, __bf16>(a, bh, d, tile, st, dry);
  }
  return hipErrorInvalidValue;
}

constexpr int kMaxStaticLds = 64 * 1024;
constexpr int kMaxLds = 160 * 1024;  // LDS per workgroup on gfx950

// More dynamic LDS than the default 64 KiB limit: the kernel's attribute has to be raised
// first, once per kernel and device (each device holds its own copy of the code object).
// Every thread keeps its own note of the (kernel, device) pairs it has done.
inline hipError_t raise_lds_limit(const void* kernel, int lds) {
  struct Note { const void* kernel; uint64_t devices; };
  constexpr int kNotes = 256;
  static thread_local Note notes[kNotes];
  static thread_local int count = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = dev < 64 ? (uint64_t)1 << dev : 0;  // (devices past 63: raised on every call)
  Note* note = nullptr;
  for (int i = 0; i < count && !note; ++i)
    if (notes[i].kernel == kernel) note = &notes[i];
  if (note && (note->devices & bit)) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return e;
  if (!note && count < kNotes) {  // (a full table: raised on every call, which is only slower)
    note = &notes[count++];
    *note = Note{kernel, 0};
  }
  if (note) note->devices |= bit;
  return hipSuccess;
}

// Launch with `lds` bytes of dynamic LDS.
template <typename Kernel, typename Args>
hipError_t launch_dyn(Kernel kernel, dim3 grid, dim3 block, int lds, hipStream_t st, const Args& a) {
  if (lds > kMaxStaticLds) {
    const hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(kernel), lds);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(kernel, grid, block, lds, st, a);
  return hipGetLastError();
}

}  // namespace tri
