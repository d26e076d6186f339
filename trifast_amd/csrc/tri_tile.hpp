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

// ---------------------------------------------------------------------------
// Swizzled LDS tiles filled by direct global->LDS loads.
//
// A tile holds ROWS rows of D elements, unpadded; the 16-byte chunks of a row are
// stored XOR-swizzled by swz(row) so that the operand reads of a wave (16 rows at
// one logical chunk, or 4 rows x 32 bytes for the transposing read) spread over
// all banks.  global_load_lds writes lane l's 16 bytes at (wave-uniform LDS base)
// + 16*l, so the swizzle costs nothing: it only decides which global address a
// lane reads.  The loads use no registers and are tracked by vmcnt; the caller
// waits with wait_dma() before the barrier that publishes the tile.
// ---------------------------------------------------------------------------
#define TRI_G1 __attribute__((address_space(1)))
#define TRI_L3 __attribute__((address_space(3)))

TRI_DEV void wait_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <typename T, int D>
struct LdsTile {
  static constexpr int ROWB = D * (int)sizeof(T);  // bytes per row
  static constexpr int CPR = ROWB / 16;            // 16-byte chunks per row (power of two)
  static constexpr int RPB = (256 / ROWB) > 0 ? 256 / ROWB : 1;  // rows per 256 bytes
  static constexpr int VEC = 16 / (int)sizeof(T);
  TRI_DEV static int swz(int r) { return (r / RPB) % CPR; }
  // byte offset, from the tile base, of byte `o` of row r (o must not straddle a chunk)
  TRI_DEV static int off(int r, int o) { return (r * CPR + ((o >> 4) ^ swz(r))) * 16 + (o & 15); }
  template <typename V>
  TRI_DEV static V read(const unsigned char* base, int r, int elem) {
    return *reinterpret_cast<const V*>(base + off(r, elem * (int)sizeof(T)));
  }
  // Fill ROWS rows; row_ptr(r) gives the global address of row r (callers clamp r
  // into range instead of branching).  NW waves share the work.
  template <int ROWS, int NW, typename RowPtr>
  TRI_DEV static void fill(unsigned char* base, RowPtr row_ptr, int wave, int lane) {
    constexpr int GROUPS = ROWS * CPR / 64;
    static_assert(ROWS * CPR % 64 == 0, "tile must be a whole number of 1 KiB wave loads");
#pragma unroll
    for (int x = 0; x < (GROUPS + NW - 1) / NW; ++x) {
      const int gi = x * NW + wave;
      if (GROUPS % NW == 0 || gi < GROUPS) {
        const int p = gi * 64 + lane;
        const int r = p / CPR, c = (p % CPR) ^ swz(r);
        const T* src = row_ptr(r) + c * VEC;
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)src, (TRI_L3 void*)(base + gi * 1024), 16, 0, 0);
      }
    }
  }
  // A/B operand with the head-dim index in-lane: row `r`, MFMA step s over d
  TRI_DEV static typename Elem<T>::frag operand(const unsigned char* base, int r, int s, int g) {
    constexpr int KP = Elem<T>::KP;
    return read<typename Elem<T>::frag>(base, r, 2 * KP * s + KP * g);
  }
  // operand with the row (contraction) index in-lane: rows base_row + cidx(KP*step .. , g),
  // column col0 + lane%32; columns >= ncols read as zero
  TRI_DEV static typename Elem<T>::frag tr_operand(const unsigned char* base, int base_row, int step, int col0, int ncols, int lane) {
    constexpr int KP = Elem<T>::KP;
    const int g = lane >> 5;
    if (col0 + (lane & 31) >= ncols) return Elem<T>::zero();
    if constexpr (KP == 1) {
      return read<float>(base, base_row + cidx(step, g), col0 + (lane & 31));
    } else {
      const int L = lane & 15, chalf = (lane >> 4) & 1;
      const int row0 = base_row + cidx(KP * step, g);
      const int col = col0 + 16 * chalf + 4 * (L & 3);
      const auto lo = lds_tr4(reinterpret_cast<const T*>(base + off(row0 + (L >> 2), col * 2)));
      const auto hi = lds_tr4(reinterpret_cast<const T*>(base + off(row0 + 4 + (L >> 2), col * 2)));
      typename Elem<T>::frag f;
#pragma unroll
      for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
      return f;
    }
  }
};

// 4-byte-per-lane variant for rows of floats (lse, delta): 64 floats per wave load
template <int COUNT, int NW, typename Ptr>
TRI_DEV void fill_floats(float* base, Ptr elem_ptr, int wave, int lane) {
  constexpr int GROUPS = COUNT / 64;
  static_assert(COUNT % 64 == 0, "whole wave loads only");
#pragma unroll
  for (int x = 0; x < (GROUPS + NW - 1) / NW; ++x) {
    const int gi = x * NW + wave;
    if (GROUPS % NW == 0 || gi < GROUPS)
      __builtin_amdgcn_global_load_lds((const TRI_G1 void*)elem_ptr(gi * 64 + lane), (TRI_L3 void*)(base + gi * 64), 4, 0, 0);
  }
}

// Two-phase version of the same copy, for software pipelining: the global loads
// of the next tile are issued into registers before the current tile is computed
// and written to LDS afterwards.
template <typename T, int D, int ROWS, int NT>
struct TileRegs {
  using vec = typename Elem<T>::vec;
  static constexpr int VEC = Elem<T>::VEC;
  static constexpr int CPR = D / VEC;
  static constexpr int CNT = (ROWS * CPR + NT - 1) / NT;
  vec v[CNT];
  TRI_DEV void load(const T* src, int64_t stride, int nrows, int tid) {
#pragma unroll
    for (int x = 0; x < CNT; ++x) {
      const int c = x * NT + tid;
      const int row = c / CPR, col = (c % CPR) * VEC;
      if (c < ROWS * CPR && row < nrows) {
        v[x] = *reinterpret_cast<const vec*>(src + (int64_t)row * stride + col);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[x][e] = (T)0.f;
      }
    }
  }
  template <int LD>
  TRI_DEV void store(T (*dst)[LD], int tid) const {
#pragma unroll
    for (int x = 0; x < CNT; ++x) {
      const int c = x * NT + tid;
      const int row = c / CPR, col = (c % CPR) * VEC;
      if (c < ROWS * CPR) *reinterpret_cast<vec*>(&dst[row][col]) = v[x];
    }
  }
};

// The packed bias operand of tile (jt, kt) for one lane: 2 x 8 elements.
template <typename T>
struct BiasRegs {
  typename Elem<T>::vec v[2 * (sizeof(T) == 2 ? 1 : 2)];
  TRI_DEV void load(const T* pack_bh, int NP, int jt, int kt, int lane_q) {
    const T* p = pack_bh + ((((int64_t)jt * NP + kt) * 2) * 64 + lane_q) * 8;
    if constexpr (sizeof(T) == 2) {
      v[0] = *reinterpret_cast<const typename Elem<T>::vec*>(p);
      v[1] = *reinterpret_cast<const typename Elem<T>::vec*>(p + 512);
    } else {
      v[0] = *reinterpret_cast<const f32x4*>(p);
      v[1] = *reinterpret_cast<const f32x4*>(p + 4);
      v[2] = *reinterpret_cast<const f32x4*>(p + 512);
      v[3] = *reinterpret_cast<const f32x4*>(p + 516);
    }
  }
  // element x (0..15) as float
  TRI_DEV float at(int x) const {
    if constexpr (sizeof(T) == 2) return (float)v[x / 8][x % 8];
    else return v[x / 4][x % 4];
  }
};

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

// The bias enters the raw scores through the matrix pipe rather than the vector
// ALU: S^T[key, j] += sum_k' (sqrt(d) * I)[key, k'] * bias^T[k', j].  The packed
// bias tile is the B operand as stored (no conversion); the A operand is the
// scaled identity, whose row m stands for key perm32(m).  sqrt(d) is split into
// hi + lo parts of the operand type so the product is exact to ~2^-17 (for d a
// power of 4 the lo part is zero and is skipped).  fp32 needs no split.
template <typename T>
struct BiasIdentity {
  using frag = typename Elem<T>::frag;
  static constexpr int KP = Elem<T>::KP;
  static constexpr int PS = 32 / (2 * KP);
  frag hi[PS], lo[PS];
  bool has_lo;
  TRI_DEV void init(float sqrt_d, int lane) {
    const int m = perm32(lane & 31), g = lane >> 5;
    const T h = (T)sqrt_d;
    const T l = (T)(sqrt_d - (float)h);
    has_lo = (float)l != 0.f;
#pragma unroll
    for (int s = 0; s < PS; ++s) {
      if constexpr (KP == 1) {
        hi[s] = (cidx(s, g) == m) ? sqrt_d : 0.f;
        lo[s] = 0.f;
      } else {
#pragma unroll
        for (int e = 0; e < KP; ++e) {
          const bool on = cidx(KP * s + e, g) == m;
          hi[s][e] = on ? h : (T)0.f;
          lo[s][e] = on ? l : (T)0.f;
        }
      }
    }
  }
};

// Adds sqrt(d) * bias tile (jt, kt) to the raw-score accumulator.  `lane_q` is
// the lane whose packed slot this lane reads: its own in the transposed-score
// kernels (the bias is the B operand), the row-permuted one in the dk/dv kernel
// (the bias is the A operand and the identity the B operand).
template <typename T, bool BIAS_IS_B>
TRI_DEV f32x16 add_bias_mfma(f32x16 acc, const BiasIdentity<T>& id, const T* pack_bh, int NP, int jt, int kt, int lane_q) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int PS = 32 / (2 * KP);
  const T* p = pack_bh + ((((int64_t)jt * NP + kt) * 2) * 64 + lane_q) * 8;
  frag bf[PS];
  if constexpr (KP == 1) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const f32x4 x0 = *reinterpret_cast<const f32x4*>(p + r * 512);
      const f32x4 x1 = *reinterpret_cast<const f32x4*>(p + r * 512 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { bf[8 * r + e] = x0[e]; bf[8 * r + 4 + e] = x1[e]; }
    }
  } else {
#pragma unroll
    for (int r = 0; r < 2; ++r) bf[r] = *reinterpret_cast<const frag*>(p + r * 512);
  }
#pragma unroll
  for (int s = 0; s < PS; ++s) {
    if constexpr (BIAS_IS_B) acc = E::mfma(id.hi[s], bf[s], acc);
    else acc = E::mfma(bf[s], id.hi[s], acc);
  }
  if constexpr (KP > 1) {
    if (id.has_lo) {
#pragma unroll
      for (int s = 0; s < PS; ++s) {
        if constexpr (BIAS_IS_B) acc = E::mfma(id.lo[s], bf[s], acc);
        else acc = E::mfma(bf[s], id.lo[s], acc);
      }
    }
  }
  return acc;
}

// Same, from bias operands already in registers.
template <typename T, bool BIAS_IS_B>
TRI_DEV f32x16 add_bias_mfma(f32x16 acc, const BiasIdentity<T>& id, const BiasRegs<T>& b) {
  using E = Elem<T>;
  static_assert(E::KP > 1, "the fp32 path adds the bias on the vector ALU");
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    if constexpr (BIAS_IS_B) acc = E::mfma(id.hi[s], b.v[s], acc);
    else acc = E::mfma(b.v[s], id.hi[s], acc);
  }
  if (id.has_lo) {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      if constexpr (BIAS_IS_B) acc = E::mfma(id.lo[s], b.v[s], acc);
      else acc = E::mfma(b.v[s], id.lo[s], acc);
    }
  }
  return acc;
}

template <typename T>
TRI_DEV f32x16 bias_tile(const BiasRegs<T>& b, float sqrt_d, float add) {
  f32x16 s;
#pragma unroll
  for (int x = 0; x < 16; ++x) s[x] = __builtin_fmaf(b.at(x), sqrt_d, add);
  return s;
}

// Additive key mask of one 32-key tile in the transposed-score layout: value v
// of lane group g is 0 when key cidx(v, g) is attended to and kNeg otherwise.
TRI_DEV f32x16 mask_tile(uint32_t keepw, int g) {
  const uint32_t myw = keepw >> (8 * g);
  f32x16 m;
#pragma unroll
  for (int v = 0; v < 16; ++v) m[v] = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? 0.f : kNeg;
  return m;
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
