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
// The same wait as an instruction the compiler knows: what it waits for no longer counts as
// in flight when the compiler places its own waits (vmcnt = 0, the other counters at maximum).
TRI_DEV void wait_dma_known() {
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");
}

// Stage hand-over for a ring of LDS buffers: wait until at most the newest
// IN_FLIGHT loads of this wave are outstanding (loads complete in issue order, so
// everything issued before them has landed in LDS) and every LDS read of the wave
// has returned, then meet the other waves.  A plain barrier instruction: the
// fence of __syncthreads() would wait for every load in flight.
template <int IN_FLIGHT>
TRI_DEV void ring_sync() {
  static_assert(IN_FLIGHT >= 0 && IN_FLIGHT <= 63, "vmcnt has 6 bits");
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(IN_FLIGHT) : "memory");
}

// SWZ_ROWS: rows that share one swizzle value (0: as many as make 256 bytes, which is what
// 16-byte operand reads of 16 rows want; a tile that is written with 16-byte stores, one row
// per lane, and only read back transposed wants 2: measured, the stores then run without
// bank conflicts, and transposing reads take whole rows, so any per-row swizzle suits them).
template <typename T, int D, int SWZ_ROWS = 0>
struct LdsTile {
  static constexpr int ROWB = D * (int)sizeof(T);  // bytes per row
  static constexpr int CPR = ROWB / 16;            // 16-byte chunks per row (power of two)
  static constexpr int RPB = SWZ_ROWS > 0 ? SWZ_ROWS : ((256 / ROWB) > 0 ? 256 / ROWB : 1);  // rows per swizzle value
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

// Lane-constant byte offsets of the operand reads of one wave.  Tiles start at
// rows that are multiples of 32 and MFMA steps move by 16 rows; neither changes
// the swizzle, so an operand read is (tile base + compile-time offset) + one of
// these registers.  fp32 operands are single elements with many steps: their
// offsets are computed where they are used.
template <typename T, int D, int SWZ_ROWS = 0>
struct OperandOffsets {
  using Tile = LdsTile<T, D, SWZ_ROWS>;
  using frag = typename Elem<T>::frag;
  static constexpr int KP = Elem<T>::KP;
  static constexpr int DS = D / (2 * KP);
  static constexpr int DM = (D + 31) / 32;
  static constexpr bool PRE = sizeof(T) == 2;
  int nat[PRE ? DS : 1];
  int tlo[PRE ? DM : 1], thi[PRE ? DM : 1];
  int row, lane;
  const unsigned char* base = nullptr;
  // `row_in_tile`: the row of a 32-row tile this lane reads as a natural operand
  TRI_DEV void init(int row_in_tile, int lane_) {
    row = row_in_tile;
    lane = lane_;
    if constexpr (PRE) {
      const int g = lane >> 5, L = lane & 15, chalf = (lane >> 4) & 1;
#pragma unroll
      for (int s = 0; s < DS; ++s) nat[s] = Tile::off(row, (2 * KP * s + KP * g) * (int)sizeof(T));
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        const int col = 32 * mt + 16 * chalf + 4 * (L & 3);
        tlo[mt] = Tile::off(8 * g + (L >> 2), col * 2);
        thi[mt] = Tile::off(8 * g + 4 + (L >> 2), col * 2);
      }
    }
  }
  // move every offset by a whole number of 32-row tiles (a wave's own part of a larger tile)
  TRI_DEV void shift(int bytes) {
    if constexpr (PRE) {
#pragma unroll
      for (int s = 0; s < DS; ++s) nat[s] += bytes;
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) { tlo[mt] += bytes; thi[mt] += bytes; }
    } else {
      row += bytes / Tile::ROWB;
    }
  }
  // make the offsets opaque to the compiler: it then keeps them in registers as they
  // are instead of rebuilding them from another instance plus a constant
  TRI_DEV void pin() {
    if constexpr (PRE) {
#pragma unroll
      for (int s = 0; s < DS; ++s) asm volatile("" : "+v"(nat[s]));
    }
  }
  // Fold the address of the workgroup's LDS block into the offsets: natural_at() then
  // reads from absolute LDS addresses, one register plus an immediate per read.
  TRI_DEV void make_absolute(const unsigned char* lds_base) {
    base = lds_base;
    if constexpr (PRE) {
      const int b0 = (int)(uintptr_t)(TRI_L3 const unsigned char*)lds_base;
#pragma unroll
      for (int s = 0; s < DS; ++s) nat[s] += b0;
    }
  }
  // natural operand of the 32-row tile `byte_offset` bytes into the block (after make_absolute)
  TRI_DEV frag natural_at(int byte_offset, int s) const {
    if constexpr (PRE) return *reinterpret_cast<TRI_L3 const frag*>((uintptr_t)(uint32_t)(nat[s] + byte_offset));
    else return Tile::operand(base + byte_offset, row, s, lane >> 5);
  }
  // natural operand (head-dim index in-lane), MFMA step s, of the 32-row tile at `tile`
  TRI_DEV frag natural(const unsigned char* tile, int s) const {
    if constexpr (PRE) return *reinterpret_cast<const frag*>(tile + nat[s]);
    else return Tile::operand(tile, row, s, lane >> 5);
  }
  // transposed operand (row index in-lane): rows cidx(KP*step.., g), column 32*mt + lane%32
  TRI_DEV frag transposed(const unsigned char* tile, int step, int mt) const {
    if constexpr (PRE) {
      if (D % 32 != 0 && 32 * mt + (lane & 31) >= D) return Elem<T>::zero();
      const unsigned char* p = tile + 16 * step * Tile::ROWB;
      const auto lo = lds_tr4(reinterpret_cast<const T*>(p + tlo[mt]));
      const auto hi = lds_tr4(reinterpret_cast<const T*>(p + thi[mt]));
      frag f;
#pragma unroll
      for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
      return f;
    } else {
      return Tile::tr_operand(tile, 0, step, 32 * mt, D, lane);
    }
  }
};

// A tile of ROWS rows that is re-filled stage after stage from rows that move
// along one tensor index: the per-lane source pointers are computed once for
// position 0 and a stage adds one wave-uniform element offset to them.
template <typename T, int D, int ROWS, int NW>
struct TileStream {
  using Tile = LdsTile<T, D>;
  static constexpr int GROUPS = ROWS * Tile::CPR / 64;
  static constexpr int XN = (GROUPS + NW - 1) / NW;
  static_assert(ROWS * Tile::CPR % 64 == 0, "tile must be a whole number of 1 KiB wave loads");
  const T* p0[XN];
  template <typename RowPtr>
  TRI_DEV void init(RowPtr row_ptr, int wave, int lane) {
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const int gi = (GROUPS % NW == 0) ? x * NW + wave : min(x * NW + wave, GROUPS - 1);
      const int p = gi * 64 + lane;
      const int r = p / Tile::CPR, c = (p % Tile::CPR) ^ Tile::swz(r);
      p0[x] = row_ptr(r) + c * Tile::VEC;
    }
  }
  // EVERY = true: a wave whose share of the tile is empty repeats the tile's last
  // piece instead of skipping it, so that every wave issues exactly XN loads (a
  // fixed count is what lets a later s_waitcnt vmcnt(k) stand for "all but the
  // newest stages have landed")
  template <bool EVERY = false>
  TRI_DEV void issue(unsigned char* base, int64_t elem_offset, int wave) const {
    // the offset is wave-uniform: pin it to scalar registers so that a stage costs
    // one 64-bit add per load
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)elem_offset);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)elem_offset >> 32));
    elem_offset = (int64_t)(((uint64_t)hi << 32) | lo);
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const int gi = EVERY ? min(x * NW + wave, GROUPS - 1) : x * NW + wave;
      if (EVERY || GROUPS % NW == 0 || gi < GROUPS)
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p0[x] + elem_offset), (TRI_L3 void*)(base + gi * 1024), 16, 0, 0);
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

// The same for COUNT floats that move along one index (lse, delta of a query tile).
template <int COUNT, int NW>
struct FloatStream {
  static constexpr int GROUPS = COUNT / 64;
  static constexpr int XN = (GROUPS + NW - 1) / NW;
  static_assert(COUNT % 64 == 0, "whole wave loads only");
  const float* p0[XN];
  template <typename Ptr>
  TRI_DEV void init(Ptr elem_ptr, int wave, int lane) {
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const int gi = (GROUPS % NW == 0) ? x * NW + wave : min(x * NW + wave, GROUPS - 1);
      p0[x] = elem_ptr(gi * 64 + lane);
    }
  }
  template <bool EVERY = false>
  TRI_DEV void issue(float* base, int64_t elem_offset, int wave) const {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)elem_offset);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)elem_offset >> 32));
    elem_offset = (int64_t)(((uint64_t)hi << 32) | lo);
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const int gi = EVERY ? min(x * NW + wave, GROUPS - 1) : x * NW + wave;
      if (EVERY || GROUPS % NW == 0 || gi < GROUPS)
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p0[x] + elem_offset), (TRI_L3 void*)(base + gi * 64), 4, 0, 0);
    }
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

// Which 32-key tiles matter to the R pair rows of a workgroup, as bitmaps over
// the key tiles, one 64-bit word per 64 tiles, built once into LDS:
//   live  = some row attends to some key of the tile (other tiles are skipped:
//           their probabilities are exactly zero),
//   plain = every row attends to every key of the tile (no mask work at all).
// The words of the 64-tile chunk in use are cached in scalar registers, so the
// per-stage queries are scalar bit operations.
// A 64-bit word that every lane holds, as a wave-uniform value (the two halves go through
// readfirstlane, whose result is a signed int: each half is widened as unsigned).
TRI_DEV uint64_t uniform_u64(uint64_t x) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)x);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(x >> 32));
  return ((uint64_t)hi << 32) | lo;
}

struct KeyTileMasks {
  const uint64_t* words;  // LDS: [nchunks] live, then [nchunks] plain
  int nchunks, ntiles, cur;
  uint64_t live, plain;

  static constexpr int lds_bytes(int nwords) { return 16 * ((nwords + 63) / 64); }

  // keep_row(r) = pointer to the keep words of row r.  Every wave calls this; the
  // caller synchronises the workgroup before the first query.
  template <int R, int NW, typename KeepRow>
  TRI_DEV void build(uint64_t* lds, KeepRow keep_row, int nwords, bool force_not_plain, int wave, int lane) {
    words = lds;
    ntiles = nwords;
    nchunks = (nwords + 63) / 64;
    cur = -1;
    live = plain = 0;
    for (int ch = wave; ch < nchunks; ch += NW) {
      const int w = ch * 64 + lane;
      uint32_t any = 0, all = 0xffffffffu;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t x = (w < nwords) ? keep_row(r)[w] : 0u;
        any |= x;
        all &= x;
      }
      const uint64_t lv = __ballot(any != 0);
      const uint64_t pl = force_not_plain ? 0 : __ballot(all == 0xffffffffu);
      if (lane == 0) {
        lds[ch] = lv;
        lds[nchunks + ch] = pl;
      }
    }
  }
  TRI_DEV void select(int ch) {
    if (ch == cur) return;
    cur = ch;
    const uint64_t lv = words[ch], pl = words[nchunks + ch];
    live = uniform_u64(lv);
    plain = uniform_u64(pl);
  }
  // first stage of KU tiles at or after tile t (t % KU == 0) with a live tile; ntiles if none
  template <int KU>
  TRI_DEV int next_live(int t) {
    while (t < ntiles) {
      select(t >> 6);
      const uint64_t m = live >> (t & 63);
      if (m != 0) {
        const int pos = __builtin_ctzll(m);
        return t + pos - pos % KU;
      }
      t = ((t >> 6) + 1) << 6;
    }
    return ntiles;
  }
  // one past the last key tile with an attended key, 0 if there is none (wave-uniform; reads
  // the bitmaps from LDS)
  TRI_DEV int last_live() const {
    int last = 0;
    for (int ch = 0; ch < nchunks; ++ch) {
      const uint64_t lv = words[ch];
      const uint64_t u = uniform_u64(lv);
      if (u != 0) last = 64 * ch + 64 - __builtin_clzll(u);
    }
    return last;
  }
  // every key tile is plain (wave-uniform; reads the bitmaps from LDS)
  TRI_DEV bool all_plain() const {
    bool all = true;
    for (int ch = 0; ch < nchunks; ++ch) {
      const int nt = min(64, ntiles - 64 * ch);
      const uint64_t want = nt == 64 ? ~0ull : ((1ull << nt) - 1);
      const uint64_t pl = words[nchunks + ch];
      const uint64_t u = uniform_u64(pl);
      all = all && (u & want) == want;
    }
    return all;
  }
  // every tile of the stage at tile t (in the chunk last selected) is plain
  template <int KU>
  TRI_DEV bool stage_plain(int t) const {
    constexpr uint64_t kMask = (1ull << KU) - 1;
    return ((plain >> (t & 63)) & kMask) == kMask;
  }
};

// Compile-time versions of a stage loop, chosen per workgroup: every row attends to
// every key (constant keys operand, no per-tile branch); some keys are masked but no
// row is fully masked (dead tiles skipped); anything.
constexpr int kPlain = 0, kMasked = 1, kGeneral = 2;

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

// The same store for 16-bit outputs with 16 bytes per lane: lane l and lane l ^ 32 own the
// two halves of every 8 columns of one row; they trade values (v_permlane32_swap) so that
// the lower lane ends up with columns 32*mt + 8*h + 0..7 and the upper lane with columns
// 32*mt + 16 + 8*h + 0..7, each whole.  Half as many store instructions, each of them
// writing whole 16-byte pieces.  Every lane of the wave takes part in the exchange;
// `active` says whether this lane's row is stored.
template <typename T, int D, int DM>
TRI_DEV void store_rows_wide(T* out_row, const f32x16* acc, float mul, int g, bool active) {
  static_assert(sizeof(T) == 2, "16-bit outputs");
  using E = Elem<T>;
  typedef uint32_t u32x2s __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int mt = 0; mt < DM; ++mt) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      typename E::vec4 lo4, hi4;  // this lane's columns 8h + 4g + 0..3 and 8(h+2) + 4g + 0..3
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo4[e] = (T)(acc[mt][4 * h + e] * mul);
        hi4[e] = (T)(acc[mt][4 * (h + 2) + e] * mul);
      }
      const u32x2s x = __builtin_bit_cast(u32x2s, lo4), y = __builtin_bit_cast(u32x2s, hi4);
      const auto r0 = __builtin_amdgcn_permlane32_swap(x[0], y[0], false, false);
      const auto r1 = __builtin_amdgcn_permlane32_swap(x[1], y[1], false, false);
      const u32x4s out = {(uint32_t)r0[0], (uint32_t)r1[0], (uint32_t)r0[1], (uint32_t)r1[1]};
      const int d0 = 32 * mt + 16 * g + 8 * h;
      if (active && d0 < D) *reinterpret_cast<u32x4s*>(out_row + d0) = out;
    }
  }
}

// either of the two, by the element type
template <typename T, int D, int DM>
TRI_DEV void store_rows_any(T* out_row, const f32x16* acc, float mul, int g, bool active) {
  if constexpr (sizeof(T) == 2) {
    store_rows_wide<T, D, DM>(out_row, acc, mul, g, active);
  } else {
    if (active) store_rows<T, D, DM>(out_row, acc, mul, g);
  }
}

}  // namespace tri
