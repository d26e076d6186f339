// Output gating of a triangle-attention block, fused with the layout change between the
// operator and the output projection:
//   forward   y[b, i, j, h, :]  = o[b, h, i, j, :] * sigmoid(g[b, i, j, h, :])
//   backward  do[b, h, i, j, :] = dy[b, i, j, h, :] * sigmoid(g[b, i, j, h, :])
//             dg[b, i, j, h, :] = dy[b, i, j, h, :] * o[b, h, i, j, :] * s (1 - s)
// o, do are in the operator's layout (heads outermost), g, dg, y, dy in the layout a linear
// layer over the pair representation produces and consumes (heads interleaved), so neither
// a permuted copy of o before the output projection nor one of do before the operator's
// backward is needed.  Streaming kernels: one 16-byte chunk of a head row per lane, fp32
// arithmetic; bound by HBM (forward 3, backward 5 tensors of b h n^2 d elements).
// No counterpart in the reference: its callers are only hinted at by the module of
// reference tests/unit/test_trifast.py:152-169.
#pragma once
#include "tri_common.hpp"

namespace tri {

struct GateArgs {
  void* y;         // forward: y; backward: dg
  void* dox;       // backward: do
  const void* o;
  const void* g;
  const void* dy;  // backward only
  int64_t rows;    // b * n * n
  int64_t plane;   // n * n
  int H, D;
};

template <typename T>
struct GateVec {
  static constexpr int VEC = 16 / (int)sizeof(T);
  typedef T type __attribute__((ext_vector_type(VEC)));
};

// sigmoid(x) and its derivative s (1 - s) from e = exp(-|x|) <= 1: no overflow, and no
// cancellation in 1 - s for large |x|.
TRI_DEV void gate_sigmoid(float x, float& s, float& ds) {
  const float e = __expf(-fabsf(x));
  const float r = 1.0f / (1.0f + e);
  s = x >= 0.0f ? r : e * r;
  ds = e * r * r;
}

template <typename T, bool BWD>
__global__ __launch_bounds__(256) void gate_kernel(const GateArgs a) {
  constexpr int VEC = GateVec<T>::VEC;
  typedef typename GateVec<T>::type vec;
  const int cpr = a.D / VEC;  // chunks per head row
  const int64_t chunks = a.rows * a.H * cpr;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < chunks; idx += (int64_t)gridDim.x * 256) {
    const int c = (int)(idx % cpr);
    const int64_t rh = idx / cpr;
    const int h = (int)(rh % a.H);
    const int64_t row = rh / a.H;  // (b, i, j)
    const int64_t b = row / a.plane, ij = row % a.plane;
    const int64_t inter = idx * VEC;                                             // heads interleaved
    const int64_t outer = (((b * a.H + h) * a.plane + ij) * a.D) + (int64_t)c * VEC;  // heads outermost
    const vec gv = *reinterpret_cast<const vec*>(reinterpret_cast<const T*>(a.g) + inter);
    const vec ov = *reinterpret_cast<const vec*>(reinterpret_cast<const T*>(a.o) + outer);
    if constexpr (!BWD) {
      vec yv;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float s, ds;
        gate_sigmoid((float)gv[e], s, ds);
        yv[e] = (T)((float)ov[e] * s);
      }
      *reinterpret_cast<vec*>(reinterpret_cast<T*>(a.y) + inter) = yv;
    } else {
      const vec dyv = *reinterpret_cast<const vec*>(reinterpret_cast<const T*>(a.dy) + inter);
      vec dov, dgv;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float s, ds;
        gate_sigmoid((float)gv[e], s, ds);
        const float d = (float)dyv[e];
        dov[e] = (T)(d * s);
        dgv[e] = (T)(d * (float)ov[e] * ds);
      }
      *reinterpret_cast<vec*>(reinterpret_cast<T*>(a.dox) + outer) = dov;
      *reinterpret_cast<vec*>(reinterpret_cast<T*>(a.y) + inter) = dgv;
    }
  }
}

template <bool BWD>
inline hipError_t gate_launch(const GateArgs& a, int dtype, hipStream_t st) {
  const int vec = dtype == kF32 ? 4 : 8;
  const int64_t chunks = a.rows * a.H * (a.D / vec);
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;  // grid-stride beyond 64 workgroups per CU
  const dim3 grid((unsigned)blocks), block(256);
  switch (dtype) {
    case kF32: hipLaunchKernelGGL((gate_kernel<float, BWD>), grid, block, 0, st, a); break;
    case kBF16: hipLaunchKernelGGL((gate_kernel<__bf16, BWD>), grid, block, 0, st, a); break;
    default: hipLaunchKernelGGL((gate_kernel<_Float16, BWD>), grid, block, 0, st, a); break;
  }
  return hipGetLastError();
}

}  // namespace tri
