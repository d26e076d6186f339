// Shared device-side pieces of the gfx950 triangle-attention kernels.
//
// MFMA register layouts used everywhere (wave64, 32x32 tiles):
//   A operand (M=32 rows x contraction): lane l supplies row l%32 and the KP
//     contraction slots owned by lane group g = l/32.
//   B operand (contraction x N=32 cols): lane l supplies column l%32, same slots.
//   C/D (32x32 fp32, 16 values per lane): value v of lane l is
//     row 8*(v/4) + 4*g + v%4, column l%32.
// A C tile can feed the next MFMA as a B (or A) operand without leaving
// registers when the contraction runs over its in-lane (row) index: slot
// (g, v) of the C tile pairs with slot (g, v) of the other operand.  To make the
// other operand a single 16-byte read, tile rows are assigned to real indices
// through a permutation: value v of group g stands for real index
//   idx(v, g) = 16*(v/8) + 8*g + v%8      (8 consecutive indices per 8 values)
// which means tile row m holds real index perm32(m) = m with bits 2 and 3
// swapped.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include <utility>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define TRI_DEV __device__ __forceinline__

namespace tri {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// Finite stand-in for "minus infinity" on raw scores: large enough that
// exp2((NEG - max) * c) is exactly 0, finite so that NEG - NEG is never NaN.
constexpr float kNeg = -1.0e30f;

TRI_DEV int perm32(int m) {  // swap bits 2 and 3
  return (m & 0x13) | ((m & 4) << 1) | ((m & 8) >> 1);
}
// real index (within a 32-tile) of C value v for lane group g
TRI_DEV constexpr int cidx(int v, int g) { return 16 * (v / 8) + 8 * g + (v % 8); }
// output row (within a 32-tile) of C value v for lane group g, no permutation
TRI_DEV constexpr int crow(int v, int g) { return 8 * (v / 4) + 4 * g + (v % 4); }

template <typename T>
struct Elem;

template <>
struct Elem<__bf16> {
  static constexpr int KP = 8;    // contraction slots per lane per MFMA
  static constexpr int VEC = 8;   // elements per 16-byte vector
  typedef bf16x8 frag;
  typedef bf16x8 vec;
  typedef bf16x4 vec4;
  // 16 contraction slots of this element sum to a "minus infinity" raw score
  static constexpr float kMaskElem = -1.0e29f;
  static TRI_DEV f32x16 mfma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // the same with the accumulator held in the accumulation registers (AGPRs): for
  // long-lived accumulators of kernels that run one wave per SIMD, whose other values
  // fill the ordinary registers.  Nothing but MFMAs touches `c` between its
  // initialisation and its final read.  The compiler does not know that the statement
  // is an MFMA, so the wait states an MFMA needs after a vector-ALU write of one of its
  // operands (two) are spent inside the statement.
  // (TRI_MFMA_ACC_BUILTIN: the same through the compiler's own MFMA, for a toolchain the asm
  // form has not been validated with: the compiler then places the accumulators and the wait
  // states itself, at the price of register copies where the register file is full)
  static TRI_DEV void mfma_acc(frag a, frag b, f32x16& c) {
#ifdef TRI_MFMA_ACC_BUILTIN
    c = mfma(a, b, c);
#else
asm("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#endif
  }
  // Such an accumulator is zeroed by an MFMA too (0 * 0 + 0): a vector-ALU write to it
  // right before the first accumulating MFMA is not ordered against that MFMA's read by
  // anything the compiler knows about an asm statement.
  static TRI_DEV void mfma_acc_zero(f32x16& c) {
#ifdef TRI_MFMA_ACC_BUILTIN
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = 0.f;
#else
    const frag z = zero();
asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=a"(c) : "v"(z));  // volatile: one MFMA per accumulator, no copies
#endif
  }
  static TRI_DEV frag splat(float x) {
    frag f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (__bf16)x;
    return f;
  }
  static TRI_DEV frag zero() { return (frag){0, 0, 0, 0, 0, 0, 0, 0}; }
  static TRI_DEV frag pack(const float* x) {
    frag r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)x[e];
    return r;
  }
};

template <>
struct Elem<_Float16> {
  static constexpr int KP = 8;
  static constexpr int VEC = 8;
  typedef f16x8 frag;
  typedef f16x8 vec;
  typedef f16x4 vec4;
  // fp16 cannot hold -1e30: 16 slots of -60000 give -9.6e5, far below any raw score
  static constexpr float kMaskElem = -60000.0f;
  static TRI_DEV f32x16 mfma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static TRI_DEV void mfma_acc(frag a, frag b, f32x16& c) {
#ifdef TRI_MFMA_ACC_BUILTIN
    c = mfma(a, b, c);
#else
    asm("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#endif
  }
  static TRI_DEV void mfma_acc_zero(f32x16& c) {
#ifdef TRI_MFMA_ACC_BUILTIN
#pragma unroll
    for (int v = 0; v < 16; ++v) c[v] = 0.f;
#else
    const frag z = zero();
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %1, 0" : "=a"(c) : "v"(z));
#endif
  }
  static TRI_DEV frag splat(float x) {
    frag f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (_Float16)x;
    return f;
  }
  static TRI_DEV frag zero() { return (frag){0, 0, 0, 0, 0, 0, 0, 0}; }
  static TRI_DEV frag pack(const float* x) {
    frag r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (_Float16)x[e];
    return r;
  }
};

template <>
struct Elem<float> {
  static constexpr int KP = 1;
  static constexpr int VEC = 4;
  typedef float frag;
  typedef f32x4 vec;
  typedef f32x4 vec4;
  static constexpr float kMaskElem = -5.0e29f;  // 2 contraction slots
  static TRI_DEV f32x16 mfma(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  static TRI_DEV frag splat(float x) { return x; }
  static TRI_DEV frag zero() { return 0.f; }
  static TRI_DEV frag pack(const float* x) { return x[0]; }
};

typedef short s16x4v __attribute__((__vector_size__(4 * sizeof(short))));
#define TRI_LDS __attribute__((address_space(3)))

// ds_read_b64_tr_b16: within each group of 16 lanes, lane L receives element e
// (0..3) from the 64 bits supplied by lane 4e + L/4, at position L%4.  With lane
// L' pointing at tile[row0 + L'/4][col0 + 4*(L'%4)], lane L ends up with
// tile[row0 + e][col0 + L]: a column of four rows, i.e. the tile read transposed.
TRI_DEV bf16x4 lds_tr4(const __bf16* p) {
  const s16x4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS s16x4v*)(p));
  return __builtin_bit_cast(bf16x4, r);
}
TRI_DEV f16x4 lds_tr4(const _Float16* p) {
  const s16x4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS s16x4v*)(p));
  return __builtin_bit_cast(f16x4, r);
}
// the same from pointers that are already in the LDS address space
TRI_DEV bf16x4 lds_tr4(TRI_LDS const __bf16* p) {
  const s16x4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS s16x4v*)(p));
  return __builtin_bit_cast(bf16x4, r);
}
TRI_DEV f16x4 lds_tr4(TRI_LDS const _Float16* p) {
  const s16x4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((TRI_LDS s16x4v*)(p));
  return __builtin_bit_cast(f16x4, r);
}

// Operand with the contraction index in-lane, read from a natural row-major LDS
// tile[rows = contraction index][cols]: the lane gets tile[row0 .. row0+7][col0 + lane%32]
// (row0 must already include the lane group's +8*g).  Two transposed reads.
template <typename T, int LD>
TRI_DEV typename Elem<T>::frag lds_tr_frag(const T (*tile)[LD], int row0, int col0, int lane) {
  static_assert(sizeof(T) == 2, "transposed LDS reads exist for 16-bit types only");
  const int L = lane & 15, chalf = (lane >> 4) & 1;
  const T* p = &tile[row0 + (L >> 2)][col0 + 16 * chalf + 4 * (L & 3)];
  const auto lo = lds_tr4(p);
  const auto hi = lds_tr4(p + 4 * LD);
  typename Elem<T>::frag f;
#pragma unroll
  for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
  return f;
}

// sum of the KP values of a packed operand, added to acc (consistent with what
// the MFMA consumes: the rounded values are what is summed)
TRI_DEV float frag_sum(bf16x8 f, float acc) {
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    const bf16x2 pr = {f[e], f[e + 1]};
    acc = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, acc, false);
  }
  return acc;
}
TRI_DEV float frag_sum(f16x8 f, float acc) {
  const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    const f16x2 pr = {f[e], f[e + 1]};
    acc = __builtin_amdgcn_fdot2(pr, ones, acc, false);
  }
  return acc;
}
TRI_DEV float frag_sum(float f, float acc) { return acc + f; }

template <typename T>
TRI_DEV float to_f32(T x) { return (float)x; }

TRI_DEV float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
TRI_DEV float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Lane l and lane l^32 hold the two halves of one column.  v_permlane32_swap
// hands every lane its own value and its partner's (in an order that depends on
// the half), which is all a max or a sum of the two needs.
TRI_DEV void half_pair(float x, float& a, float& b) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  a = __builtin_bit_cast(float, (unsigned)r[0]);
  b = __builtin_bit_cast(float, (unsigned)r[1]);
}
TRI_DEV float half_max(float x) { float a, b; half_pair(x, a, b); return fmaxf(a, b); }
TRI_DEV float half_sum(float x) { float a, b; half_pair(x, a, b); return a + b; }

// Per-row (or per-column) additive terms through the matrix pipe: acc[m][n] += x[m]
// is one extra MFMA whose A operand holds x[m] in its first contraction slots and
// whose B operand is all ones (or the other way round for a per-column term).
// For the 16-bit types x is split into hi + lo parts (two slots), which keeps
// 16 / 22 significant bits; fp32 needs one slot.  split_word() packs the parts
// into one 32-bit word (so they can be stored per query by one kernel and loaded
// by another); rank1_operand() turns the word into the operand of the lane that
// owns row / column m: lanes of group 0 supply the first slots, group 1 zeros.
template <typename T>
TRI_DEV uint32_t split_word(float x) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(uint32_t, x);
  } else {
    const T hi = (T)x;
    const T lo = (T)(x - (float)hi);
    return (uint32_t)__builtin_bit_cast(uint16_t, hi) | ((uint32_t)__builtin_bit_cast(uint16_t, lo) << 16);
  }
}
// the number a split word stands for
template <typename T>
TRI_DEV float split_value(uint32_t w) {
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(float, w);
  } else {
    const T hi = __builtin_bit_cast(T, (uint16_t)(w & 0xffffu));
    const T lo = __builtin_bit_cast(T, (uint16_t)(w >> 16));
    return (float)hi + (float)lo;
  }
}
// Per-query offset and key mask through ONE extra MFMA of a transposed score tile
// (rows = keys, columns = queries): the contraction slots are shared between the two
// rank-1 terms.
//   slots of dword 0 of lane group 0: keys operand 1,      queries operand: split word
//   slots of dword 1 of every lane:   keys operand: mask element of the key (or 0),
//                                     queries operand 1
// (fp32 has one slot per lane group: group 0 carries the offset, group 1 the mask.)
// Both operands are kept in place: per tile only the mask dword of the keys operand
// changes, and the word of the queries operand changes when the offset does.
template <typename T>
struct OffsetMask {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef typename Elem<T>::frag frag;
  static TRI_DEV uint32_t ones_dword() {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(uint32_t, 1.0f);
    else return (uint32_t)__builtin_bit_cast(uint16_t, (T)1.0f) * 0x10001u;
  }
  static TRI_DEV uint32_t mask_dword() {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(uint32_t, Elem<T>::kMaskElem);
    else return (uint32_t)__builtin_bit_cast(uint16_t, (T)Elem<T>::kMaskElem) * 0x10001u;
  }
  static TRI_DEV frag as_frag(u32x4 v) {
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(float, v[0]);
    else return __builtin_bit_cast(frag, v);
  }
  // keys operand of the lane whose operand row stands for key `key_in_tile`
  struct Keys {
    u32x4 v;
    uint32_t bit;
    int g;
    TRI_DEV void init(int key_in_tile, int g_) {
      g = g_;
      bit = 1u << key_in_tile;
      v = u32x4{g ? 0u : ones_dword(), 0u, 0u, 0u};
    }
    // no key of the tile is masked
    TRI_DEV frag plain() const { return as_frag(v); }
    // bit k of keepw set = key k of the tile is attended
    TRI_DEV frag masked(uint32_t keepw) {
      const uint32_t m = (keepw & bit) ? 0u : mask_dword();
      if constexpr (sizeof(T) == 4) {
        u32x4 t = v;
        if (g) t[0] = m;
        return as_frag(t);
      } else {
        v[1] = m;
        return as_frag(v);
      }
    }
    // the same as a new value: for callers whose tiles are rarely masked (the operand in
    // place would be carried, and copied, through the unmasked path as well)
    TRI_DEV frag masked_copy(uint32_t keepw) const {
      const uint32_t m = (keepw & bit) ? 0u : mask_dword();
      u32x4 t = v;
      if constexpr (sizeof(T) == 4) {
        if (g) t[0] = m;
      } else {
        t[1] = m;
      }
      return as_frag(t);
    }
  };
  // queries operand of the lane that owns a query
  struct Queries {
    u32x4 v;
    TRI_DEV void init(uint32_t word, int g) {
      if constexpr (sizeof(T) == 4) v = u32x4{g ? ones_dword() : word, 0u, 0u, 0u};
      else v = u32x4{g ? 0u : word, ones_dword(), 0u, 0u};
    }
    TRI_DEV void set(uint32_t word, int g) {
      if (!g) v[0] = word;
    }
    // `word` already holds what lanes 32..63 need (zero; fp32: one)
    TRI_DEV void set_raw(uint32_t word) { v[0] = word; }
    TRI_DEV frag get() const { return as_frag(v); }
  };
};

// The operand is kept in one variable whose first dword is replaced per use
// (rank1_set), so that the zero slots are written once and not per tile.
template <typename T>
struct Rank1 {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  u32x4 v;
  TRI_DEV void init() { v = u32x4{0u, 0u, 0u, 0u}; }
  TRI_DEV typename Elem<T>::frag set(uint32_t word, int g) { return set(g ? 0u : word); }
  // `word` is already zero in lanes 32..63
  TRI_DEV typename Elem<T>::frag set(uint32_t word) {
    v[0] = word;
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(float, v[0]);
    else return __builtin_bit_cast(typename Elem<T>::frag, v);
  }
};
template <typename T>
TRI_DEV typename Elem<T>::frag rank1_operand(uint32_t word, int g) {
  Rank1<T> r;
  r.init();
  return r.set(word, g);
}

// A fragment of ones that the compiler keeps in registers (it would otherwise
// rebuild the four registers from a constant at every use).
template <typename T>
TRI_DEV typename Elem<T>::frag resident_ones() {
  typename Elem<T>::frag f = Elem<T>::splat(1.0f);
  if constexpr (sizeof(T) == 4) {
    asm volatile("" : "+v"(f));
  } else {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v = __builtin_bit_cast(u32x4, f);
    asm volatile("" : "+v"(v));
    f = __builtin_bit_cast(typename Elem<T>::frag, v);
  }
  return f;
}

template <typename F, int... I>
TRI_DEV void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, typename F>
TRI_DEV void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// A 32-bit word at a wave-uniform index, read through the scalar cache: for words that an
// earlier kernel wrote (the scalar cache starts every kernel empty).  Several such loads are
// all in flight before the first of them is waited for, and none of them waits for vector
// memory operations in flight; a vector load followed by readfirstlane waits for everything.
TRI_DEV uint32_t uniform_word(const uint32_t* p, int idx) {
  typedef const uint32_t __attribute__((address_space(4))) * const_ptr;
  return ((const_ptr)(uintptr_t)p)[__builtin_amdgcn_readfirstlane(idx)];
}

// acc + the two values of a packed pair (what an MFMA that consumes the pair sees)
TRI_DEV float pair_sum(bf16x2 w, bf16x2 ones, float acc) { return __builtin_amdgcn_fdot2_f32_bf16(w, ones, acc, false); }
TRI_DEV float pair_sum(f16x2 w, f16x2 ones, float acc) { return __builtin_amdgcn_fdot2(w, ones, acc, false); }

TRI_DEV f32x16 zero16() {
  f32x16 z;
#pragma unroll
  for (int v = 0; v < 16; ++v) z[v] = 0.f;
  return z;
}

}  // namespace tri
