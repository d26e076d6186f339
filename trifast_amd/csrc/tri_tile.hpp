// Tile-level building blocks shared by the four kernels.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"

namespace tri {

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has
// its own L2.  All blocks that share one pair row (same K/V rows) should land on
// one XCD: with gx blocks per row, linear id L = 8*slot + xcd is re-read as
//   x = slot % gx,  y = 8 * (slot / gx) + xcd
// The launcher pads the row count to a multiple of 8; y >= rows means "no work".
TRI_DEV void xcd_remap(int gx, int& x, int& y) {
  const int L = blockIdx.x + gx * blockIdx.y;
  const int xcd = L & 7, slot = L >> 3;
  x = slot % gx;
  y = 8 * (slot / gx) + xcd;
}

// Cooperative copy of a [ROWS x D] row-major tile (row stride `stride` elements,
// rows >= nrows read as zero) into LDS in natural layout.
template <typename T, int D, int ROWS, int LD, int NT>
TRI_DEV void lds_load_natural(T (*dst)[LD], const T* src, int64_t stride, int nrows, int tid) {
  using E = Elem<T>;
  constexpr int VEC = E::VEC;
  constexpr int CPR = D / VEC;  // 16-byte chunks per row
#pragma unroll
  for (int c0 = 0; c0 < ROWS * CPR; c0 += NT) {
    const int c = c0 + tid;
    if ((ROWS * CPR) % NT != 0 && c >= ROWS * CPR) break;
    const int row = c / CPR, col = (c % CPR) * VEC;
    typename E::vec val;
    if (row < nrows) {
      val = *reinterpret_cast<const typename E::vec*>(src + (int64_t)row * stride + col);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) val[e] = (T)0.f;
    }
    *reinterpret_cast<typename E::vec*>(&dst[row][col]) = val;
  }
}

// The 16 bias values of one lane for tile (jt, kt), in the raw-score domain
// (times sqrt(d)) plus a per-lane additive term, from a packed bias array.
template <typename T>
TRI_DEV f32x16 bias_tile(const T* pack_bh, int NP, int jt, int kt, int lane, float sqrt_d, float add) {
  const T* p = pack_bh + ((((int64_t)jt * NP + kt) * 2) * 64 + lane) * 8;
  f32x16 s;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    if constexpr (sizeof(T) == 2) {
      const typename Elem<T>::vec x = *reinterpret_cast<const typename Elem<T>::vec*>(p + r * 512);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[8 * r + e] = __builtin_fmaf((float)x[e], sqrt_d, add);
    } else {
      const f32x4 x0 = *reinterpret_cast<const f32x4*>(p + r * 512);
      const f32x4 x1 = *reinterpret_cast<const f32x4*>(p + r * 512 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s[8 * r + e] = __builtin_fmaf(x0[e], sqrt_d, add);
        s[8 * r + 4 + e] = __builtin_fmaf(x1[e], sqrt_d, add);
      }
    }
  }
  return s;
}

// Operand whose contraction index is in-lane, from a natural LDS tile
// tile[contraction index][column]: 16-bit types use the transposing read, fp32
// operands are single elements.  `step` is the MFMA step within a 32-wide block
// of contraction indices starting at row `base`; the lane's column is col0 + lane%32
// (columns >= ncols read as zero).
template <typename T, int LD>
TRI_DEV typename Elem<T>::frag tr_operand(const T (*tile)[LD], int base, int step, int col0, int ncols, int lane) {
  constexpr int KP = Elem<T>::KP;
  const int g = lane >> 5;
  if (col0 + (lane & 31) >= ncols) return Elem<T>::zero();
  if constexpr (KP == 1) {
    return tile[base + cidx(step, g)][col0 + (lane & 31)];
  } else {
    return lds_tr_frag<T, LD>(tile, base + cidx(KP * step, g), col0, lane);
  }
}

// Store a 32-row tile of an [n x D] output held transposed in registers
// (lane owns row `row`, values are columns 32*mt + 8*a4 + 4*g + 0..3), scaled.
template <typename T, int D, int DM>
TRI_DEV void store_rows(T* out_row, const f32x16* acc, float mul, int g) {
  using E = Elem<T>;
#pragma unroll
  for (int mt = 0; mt < DM; ++mt) {
#pragma unroll
    for (int a4 = 0; a4 < 4; ++a4) {
      const int d0 = 32 * mt + 8 * a4 + 4 * g;
      if (d0 < D) {
        typename E::vec4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (T)(acc[mt][4 * a4 + e] * mul);
        *reinterpret_cast<typename E::vec4*>(out_row + d0) = ov;
      }
    }
  }
}

}  // namespace tri
