// Backward kernel 3 of 3: db[j, k] = sum over rows i of dS[i, j, k].
//
// Work unit: (batch*head, chunk of pair rows i, block of GJ*WJ*32 queries j, block
// of GK*WK*32 keys k).  The GJ x GK waves of a workgroup each own WJ x WK tiles of
// 32 x 32 and keep their db tiles in fp32 registers while the workgroup walks the
// rows of its chunk, so the reduction over i has one fixed order and needs no
// atomics.  Per row the workgroup stages the Q, dO rows of its queries and the K,
// V rows of its keys in LDS (direct global->LDS loads into a ring of row buffers
// that runs several rows ahead of the compute, swizzled tiles) together with
// the lse and delta operand words left by the dq kernel, and each wave
// recomputes for its tiles
//   S^T = K Q^T + bias - lse, P^T = exp2(c S^T), dP^T = V dO^T - delta, dS^T = P^T dP^T
// with every operand in its natural row-major layout: a lane owns one query
// (column) and 16 keys of each tile.  The additive terms cost the vector ALU nothing:
// the bias tiles (register-resident, fp32, raw-score domain) are the accumulator
// init of every row's score MFMA; -delta (per query) enters through one extra MFMA
// (see rank1_operand); -lse is one number per lane and is the addend of the fma that
// scales the score for exp2.  That leaves two fmas and one exp2 per element.  In a tile
// with masked keys -lse moves to an extra MFMA that it shares with the key mask (see
// OffsetMask): masked keys get a large negative score there.
//
// Waves that own two key tiles walk the plain rows at the start of a chunk as a hand-made
// software pipeline (matrix instructions of one tile between the vector instructions of the
// tile before it, operands a row ahead); see kPipelined below.
//
// All workgroups of one (batch*head, chunk) read the same rows at about the same
// time; the block index is remapped so that they run on one XCD and share its L2.
// When the rows are split into several chunks (to fill the GPU), each chunk writes
// an fp32 partial and a second kernel adds the partials in chunk order.
//
// Replaces _bwd_b of reference src/trifast/triton.py:394-501.
#pragma once
#include <type_traits>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

// -DTRI_DB_TIMING builds the kernel as a probe of its pipelined walk
// (benchmark/microbench/db_timeline.py): every wave reads the shader clock around the counted
// wait and the barrier that end a row, and leaves per wave {clocks of the walk, clocks in the
// wait, clocks in the barrier, 100 MHz ticks of the walk} where the db argument points; db
// itself is not written.  -DTRI_DB_TIMING_LOADS=0 also takes the walk's global loads out (the
// rows in LDS are then stale), =2 makes them read one row over and over (the same traffic from
// L2 to LDS, none from memory): what the loads cost the arithmetic beside them.
#if defined(TRI_DB_TIMING) && !defined(TRI_DB_TIMING_LOADS)
#define TRI_DB_TIMING_LOADS 1
#endif

namespace tri {

// LDS bytes of one stage (one pair row) of the kernel below
constexpr int bwd_b_stage_bytes(int BJ, int BKB, int ROWB) { return 2 * (BJ * 4 + 256) + (2 * BJ + 2 * BKB) * ROWB; }

template <typename T, int D, int GJ, int GK, int WJ, int WK, int NBUF>
__global__ __launch_bounds__(GJ * GK * 64) void tri_bwd_b_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int NW = GJ * GK;
  constexpr int BJ = GJ * WJ * 32, BKB = GK * WK * 32;  // queries / keys per workgroup
  constexpr int ROWB = Tile::ROWB;
  // one stage: lse2[BJ] | 64 spare words | -delta[BJ] | 64 spare words | Q rows | dO rows |
  // K rows | V rows.  The small arrays come first so that their offsets in every ring
  // buffer fit the 16-bit immediate of an LDS read.  (The row's flag and keep words do not
  // pass through LDS: they are wave-uniform and come by scalar loads.)
  constexpr int OFF_LSE = 0, OFF_DELTA = OFF_LSE + BJ * 4 + 256;
  constexpr int OFF_Q = OFF_DELTA + BJ * 4 + 256, OFF_DO = OFF_Q + BJ * ROWB, OFF_K = OFF_DO + BJ * ROWB, OFF_V = OFF_K + BKB * ROWB;
  constexpr int STAGE = OFF_V + BKB * ROWB;
  static_assert(STAGE == bwd_b_stage_bytes(BJ, BKB, ROWB), "the launcher sizes LDS with bwd_b_stage_bytes");

  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int jl = lane & 31, g = lane >> 5;
  const int N = a.N;

  // Linear block id L = 8 * slot + xcd (workgroups go to the 8 XCDs round-robin).
  // Every XCD walks its own sequence of (batch*head, chunk) groups; the launcher
  // pads the group count to a multiple of 8.
  // With fewer than 8 groups each group gets 8 / groups XCDs (whole number) and deals its
  // blocks to them in turn, so that no XCD stays idle: the rows are then fetched once per XCD
  // of the group.
  const int per_group = gridDim.x * gridDim.y;
  const int L = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const int slot = L >> 3;
  const int ngroups = a.BH * a.nchunks;
  const int share = ngroups >= 8 ? 1 : 8 / ngroups;  // XCDs per group
  const int group = share == 1 ? 8 * (slot / per_group) + (L & 7) : (L & 7) / share;
  const int within = share == 1 ? slot % per_group : slot * share + (L & 7) % share;
  if (group >= ngroups || within >= per_group) return;
  const int bh = group % a.BH, chunk = group / a.BH;
  const int b = bh / a.H, h = bh % a.H;
  const int j_blk = (within % gridDim.x) * BJ, k_blk = (within / gridDim.x) * BKB;
  const int wj = wave % GJ, wk = wave / GJ;
  const int j_wave = j_blk + wj * (WJ * 32), k_wave = k_blk + wk * (WK * 32);
  const int i_begin = chunk * a.rows_per_chunk;
  const int i_end = min(N, i_begin + a.rows_per_chunk);
  const int nrows = i_end - i_begin;

  const T* qbase = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbase = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbase = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobase = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse2_bh = reinterpret_cast<const float*>(a.lse2) + (int64_t)bh * N * N;    // 32-bit words, moved as floats
  const float* delta_bh = reinterpret_cast<const float*>(a.delta) + (int64_t)bh * N * N;

  // bias tiles in the raw-score domain: accumulator init of every row's score MFMA
  f32x16 biasr[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk)
      biasr[tj][tk] = bias_tile<T>(pack_bh, a.NP, min((j_wave >> 5) + tj, a.NP - 1), min((k_wave >> 5) + tk, a.NP - 1), lane, a.sqrt_d, 0.f);

  f32x16 dbacc[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) dbacc[tj][tk] = zero16();

  // The loads of one row, as two lists of wave-sized items: 1 KiB pieces of the Q, dO, K,
  // V tiles (16 bytes per lane), and 64-float pieces of lse2 and -delta (4 bytes per lane).  Wave w takes items w, w + NW, ...
  // of each list; every wave issues exactly XW wide and XF narrow loads per row, in that
  // order (a wave that runs out repeats the last item of the list, which rewrites the same
  // bytes), so the width of a load is known at compile time and "all but the newest K rows
  // have landed" is one s_waitcnt vmcnt(K * XN) for every wave.  Queries and keys past
  // the end are clamped (they feed db entries that are never stored).
  constexpr int CPR = Tile::CPR;
  constexpr int GQ = BJ * CPR / 64, GKK = BKB * CPR / 64, GF = BJ / 64;
  constexpr int TOTW = 2 * GQ + 2 * GKK, TOTF = 2 * GF;
  constexpr int XW = (TOTW + NW - 1) / NW, XF = (TOTF + NW - 1) / NW;
  constexpr int XN = XW + XF;
  static_assert(BJ * CPR % 64 == 0 && BKB * CPR % 64 == 0 && BJ % 64 == 0, "whole wave loads only");
  auto uniform64 = [](int64_t x) -> int64_t {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)x), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)x >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
  };
  // An item's source is a 64-bit base (wave-uniform, scalar registers, stepped from one pair
  // row to the next with scalar adds) plus a 32-bit byte offset per lane that never changes.
  const char* item_base[XN];
  uint32_t item_voff[XN];
  int64_t item_step[XN];      // bytes from one pair row to the next (wave-uniform)
  int item_lds[XN];           // destination offset inside a stage (wave-uniform)
  // (items 0 .. XW-1 move 16 bytes per lane, items XW .. XN-1 4 bytes)
  {
    const int es = (int)sizeof(T);
    auto tile_item = [&](int x, int gi, const T* base, int64_t srow, int64_t si, int blk, int off) {
      const int p = gi * 64 + lane;
      const int r = p / CPR, cc = (p % CPR) ^ Tile::swz(r);
      item_base[x] = reinterpret_cast<const char*>(uniform64((int64_t)(uintptr_t)(base + (int64_t)blk * srow + (int64_t)i_begin * si)));
      item_voff[x] = (uint32_t)(min(r, N - 1 - blk) * (int)srow + cc * Tile::VEC) * (uint32_t)es;
      item_step[x] = uniform64(si * es);
      item_lds[x] = off + gi * 1024;
    };
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      // position in the flat order Q | dO | K | V | lse2 | delta
      const int it = x < XW ? __builtin_amdgcn_readfirstlane(min(x * NW + wave, TOTW - 1))
                            : TOTW + __builtin_amdgcn_readfirstlane(min((x - XW) * NW + wave, TOTF - 1));
      if (it < GQ) {
        tile_item(x, it, qbase, a.sq.j, a.sq.i, j_blk, OFF_Q);
      } else if (it < 2 * GQ) {
        tile_item(x, it - GQ, dobase, a.sdo.j, a.sdo.i, j_blk, OFF_DO);
      } else if (it < 2 * GQ + GKK) {
        tile_item(x, it - 2 * GQ, kbase, a.sk.j, a.sk.i, k_blk, OFF_K);
      } else if (it < 2 * GQ + 2 * GKK) {
        tile_item(x, it - 2 * GQ - GKK, vbase, a.sv.j, a.sv.i, k_blk, OFF_V);
      } else {
        const int f = it - 2 * GQ - 2 * GKK;
        const int gi = f % GF;
        const float* base = (f < GF) ? lse2_bh : delta_bh;
        const int j0 = min(j_blk + gi * 64, N - 1);
        item_base[x] = reinterpret_cast<const char*>(uniform64((int64_t)(uintptr_t)(base + (int64_t)i_begin * N + j0)));
        item_voff[x] = (uint32_t)(min(lane, N - 1 - j0) * 4);
        item_step[x] = uniform64((int64_t)N * 4);
        item_lds[x] = ((f < GF) ? OFF_LSE : OFF_DELTA) + gi * 256;
      }
    }
  }
  // all ones if x > 0, else zero, as a 64-bit scalar (written out: the compiler would keep the
  // condition as a lane mask and turn it into a number with vector instructions in every row)
  auto ones_while_positive = [](int x) -> int64_t {
    int64_t m;
    asm volatile("s_cmp_gt_i32 %1, 0\n\ts_cselect_b64 %0, -1, 0" : "=s"(m) : "s"(__builtin_amdgcn_readfirstlane(x)) : "scc");
    return m;
  };
  // issue the loads of the next row into stage buffer `buf`; past the last row of
  // the chunk the bases stop and the last row is loaded again (never used)
  int rows_issued = 0;
  auto issue_row = [&](int buf) {
    const uint32_t st = (uint32_t)(uintptr_t)(TRI_L3 unsigned char*)(tri_smem + buf * STAGE);
    const int64_t advance = ones_while_positive(nrows - 1 - rows_issued);
    ++rows_issued;
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const uint32_t dst = __builtin_amdgcn_readfirstlane(st + (uint32_t)item_lds[x]);
      if (x < XW) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(item_voff[x]), "s"(item_base[x]) : "memory", "m0");
      else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(dst), "v"(item_voff[x]), "s"(item_base[x]) : "memory", "m0");
      item_base[x] += advance & item_step[x];
    }
  };
  // the same, one item at a time (for loops that deal the loads of a row between other work);
  // next_row_advance() once per row, before its items
  auto next_row_advance = [&]() __attribute__((always_inline)) -> int64_t {
#if defined(TRI_DB_TIMING) && TRI_DB_TIMING_LOADS == 2
    const int64_t advance = ones_while_positive(0);
#else
    const int64_t advance = ones_while_positive(nrows - 1 - rows_issued);
#endif
    ++rows_issued;
    return advance;
  };
  auto issue_item = [&](int buf, auto x_tag, int64_t advance) __attribute__((always_inline)) {
    constexpr int x = decltype(x_tag)::value;
    const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(TRI_L3 unsigned char*)(tri_smem + buf * STAGE) + (uint32_t)item_lds[x]);
    if constexpr (x < XW) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(item_voff[x]), "s"(item_base[x]) : "memory", "m0");
    else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(dst), "v"(item_voff[x]), "s"(item_base[x]) : "memory", "m0");
    item_base[x] += advance & item_step[x];
  };
  // wait until at most the newest `K` rows of this wave's loads are in flight and
  // every LDS read has returned, then meet the other waves
  auto sync_rows = [&](auto k_tag) {
    constexpr int K = decltype(k_tag)::value * XN;
    static_assert(K <= 63, "vmcnt has 6 bits");
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(K) : "memory");
  };

  // lane-constant LDS offsets: K, V rows as A operands (tile row m stands for key
  // perm32(m)); Q, dO rows as B operands (the lane's own query)
  OperandOffsets<T, D> ofk, ofq;
  ofk.init(perm32(jl), lane);
  ofq.init(jl, lane);
  // the wave's own tiles inside the workgroup's rows: folded into the offsets once
  ofk.shift(wk * WK * 32 * ROWB);
  ofq.shift(wj * WJ * 32 * ROWB);
  // (absolute LDS addresses from here on: the block's address is folded in once)
  ofk.make_absolute(tri_smem);
  ofq.make_absolute(tri_smem);
  ofk.pin();
  ofq.pin();
  // this lane's query in the lse / delta words, as an absolute LDS address (both halves of
  // the wave read the word of their query: lanes 32..63 zero it where it becomes a rank-1
  // operand, and use it as it is where -lse enters as a per-lane term of the exponent)
  int scalar_off = ((wj * WJ) * 32 + jl) * 4 + (int)(uintptr_t)(TRI_L3 const unsigned char*)tri_smem;
  asm volatile("" : "+v"(scalar_off));
  // (the lse word shares its MFMA with the key mask: in fp32 the slot of lanes 32..63
  // belongs to the mask and the queries operand holds a one there)
  const uint32_t upper_l = sizeof(T) == 4 ? OffsetMask<T>::ones_dword() : 0u;
  // LDS reads take a 16-bit immediate offset: for ring buffers past the first 64 KiB a
  // second set of lane offsets, moved up by two stages, keeps the buffer's offset an
  // immediate (the reads of those buffers would otherwise each need an address add)
  constexpr bool kHighSet = NBUF > 2 && sizeof(T) == 2;
  constexpr int HIGH = kHighSet ? 2 * STAGE : 0;
  OperandOffsets<T, D> ofk_hi = ofk, ofq_hi = ofq;
  int scalar_off_hi = scalar_off;
  if constexpr (kHighSet) {
    ofk_hi.shift(HIGH);
    ofq_hi.shift(HIGH);
    ofk_hi.pin();
    ofq_hi.pin();
    scalar_off_hi += HIGH;
    asm volatile("" : "+v"(scalar_off_hi));
  }
  const frag ones = resident_ones<T>();
  // -lse per query and the key mask share one MFMA (see OffsetMask), -delta has its own
  typename OffsetMask<T>::Queries lrank[WJ];
  Rank1<T> drank[WJ];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj) { lrank[tj].init(0u, g); drank[tj].init(); }
  typename OffsetMask<T>::Keys kop;
  kop.init(perm32(jl), g);

  const float c = a.c;
  // (an integer that the compiler cannot see through: a boolean would be kept as a lane mask
  // and negated with vector instructions in every row)
  int wave_live = __builtin_amdgcn_readfirstlane((int)(j_wave < N && k_wave < N));
  asm volatile("" : "+s"(wave_live));

  // The row's flag and the keep words of the wave's key tiles are the same for every lane:
  // they are read from global memory with scalar loads, one row ahead of their use (rows
  // past the end of the chunk repeat the last one and are not used).
  struct RowMeta {
    uint32_t flag;
    uint32_t keep[WK];
  };
  typedef const __attribute__((address_space(4))) uint32_t* const_words;
  const int64_t keep_step = uniform64((int64_t)a.nwords * 4);
  const_words flag_word = (const_words)(uintptr_t)(a.rowflag + (int64_t)b * N + i_begin);
  // (a key tile past the last word of the row has no attended key: its word is never read)
  const_words keep_word = (const_words)(uintptr_t)(a.keep + ((int64_t)b * N + i_begin) * a.nwords + min(k_wave / 32, a.nwords - 1));
  int word_at[WK];         // offset of tile tk's word from keep_word (clamped to the row)
  uint32_t word_mask[WK];  // zero for a tile past the last word
#pragma unroll
  for (int tk = 0; tk < WK; ++tk) {
    word_at[tk] = __builtin_amdgcn_readfirstlane(min(k_wave / 32 + tk, a.nwords - 1) - min(k_wave / 32, a.nwords - 1));
    word_mask[tk] = __builtin_amdgcn_readfirstlane(k_wave / 32 + tk < a.nwords ? 0xffffffffu : 0u);
  }
  int meta_rows = 0;
  // the words of the next row (the first call gives those of row 0)
  auto load_meta = [&]() -> RowMeta {
    RowMeta m;
    m.flag = *flag_word;
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) m.keep[tk] = keep_word[word_at[tk]] & word_mask[tk];
    const int64_t advance = ones_while_positive(nrows - 1 - meta_rows);
    ++meta_rows;
    flag_word = (const_words)((uintptr_t)flag_word + (uintptr_t)(advance & 4));
    keep_word = (const_words)((uintptr_t)keep_word + (uintptr_t)(advance & keep_step));
    return m;
  };

  auto compute_row = [&](int buf, const RowMeta& meta) __attribute__((always_inline)) {
    const bool high = kHighSet && buf >= 2;  // (a constant once the ring loop is unrolled)
    const int sl = buf * STAGE - (high ? HIGH : 0);  // offset of the buffer for reads through the lane offsets
    const OperandOffsets<T, D>& oq = high ? ofq_hi : ofq;
    const OperandOffsets<T, D>& ok = high ? ofk_hi : ofk;
    const int soff = high ? scalar_off_hi : scalar_off;
    // (wave-uniform values are pinned to scalar registers so that the branches on
    // them are real branches and not lane masks)
    const bool flagged = meta.flag != 0;
    frag qf[WJ][DS], dof[WJ][DS], kf[WK][DS], vf[WK][DS];
    frag lf[WJ], df[WJ];  // per-query terms -lse*sqrt(d) and -delta as rank-1 MFMA operands
    float nl2[WJ];         // -lse of this lane's query in the exponent's unit
    uint32_t lw[WJ], dw[WJ];
#pragma unroll
    for (int tj = 0; tj < WJ; ++tj) {
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        qf[tj][s] = oq.natural_at(sl + OFF_Q + tj * 32 * ROWB, s);
        dof[tj][s] = oq.natural_at(sl + OFF_DO + tj * 32 * ROWB, s);
      }
      lw[tj] = *reinterpret_cast<TRI_L3 const uint32_t*>((uintptr_t)(uint32_t)(sl + OFF_LSE + tj * 128 + soff));
      dw[tj] = *reinterpret_cast<TRI_L3 const uint32_t*>((uintptr_t)(uint32_t)(sl + OFF_DELTA + tj * 128 + soff));
    }
#pragma unroll
    for (int tk = 0; tk < WK; ++tk)
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        kf[tk][s] = ok.natural_at(sl + OFF_K + tk * 32 * ROWB, s);
        vf[tk][s] = ok.natural_at(sl + OFF_V + tk * 32 * ROWB, s);
      }
    // every LDS read of the row is issued before the first branch on the row's keep words
    // (read where they are used, they would return in several waited-for batches)
#pragma unroll
    for (int tj = 0; tj < WJ; ++tj) {
#pragma unroll
      for (int s = 0; s < DS; ++s) asm volatile("" : "+v"(qf[tj][s]), "+v"(dof[tj][s]));
      asm volatile("" : "+v"(lw[tj]), "+v"(dw[tj]));
    }
#pragma unroll
    for (int tk = 0; tk < WK; ++tk)
#pragma unroll
      for (int s = 0; s < DS; ++s) asm volatile("" : "+v"(kf[tk][s]), "+v"(vf[tk][s]));
#pragma unroll
    for (int tj = 0; tj < WJ; ++tj) {
      lrank[tj].set_raw(g ? upper_l : lw[tj]);
      lf[tj] = lrank[tj].get();
      df[tj] = drank[tj].set(g ? 0u : dw[tj]);
      nl2[tj] = split_value<T>(lw[tj]) * c;
    }
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
      const uint32_t keepw = meta.keep[tk];
      if (keepw == 0) continue;  // no attended key in this tile: dS = 0
#pragma unroll
      for (int tj = 0; tj < WJ; ++tj) {
        f32x16 s;
        float addend = 0.f;
        // Each case ends in the MFMA that defines s from the bias tile in place (a
        // select between accumulator inits would copy 16 registers).
        if (!flagged) {
          if (keepw == 0xffffffffu) {
            // no masked key in the tile: a lane owns one query, so -lse is one number per
            // lane and rides on the multiply of the exponent (an fma) instead of an MFMA
            s = E::mfma(kf[tk][0], qf[tj][0], biasr[tj][tk]);
#pragma unroll
            for (int sd = 1; sd < DS; ++sd) s = E::mfma(kf[tk][sd], qf[tj][sd], s);
            addend = nl2[tj];
          } else {
            s = E::mfma(kop.masked_copy(keepw), lf[tj], biasr[tj][tk]);  // masked keys: large negative score
#pragma unroll
            for (int sd = 0; sd < DS; ++sd) s = E::mfma(kf[tk][sd], qf[tj][sd], s);
          }
        } else {
          // rare: a fully masked row ignores q.k and the bias
          asm volatile("" ::);
          s = E::mfma(kop.masked_copy(keepw), lf[tj], zero16());
        }
        f32x16 dp = E::mfma(ones, df[tj], zero16());
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) dp = E::mfma(vf[tk][sd], dof[tj][sd], dp);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = fast_exp2(__builtin_fmaf(s[v], c, addend));
          dbacc[tj][tk][v] = __builtin_fmaf(p, dp[v], dbacc[tj][tk][v]);
        }
      }
    }
  };

  // the rows from `first_row` on (the loads and the row words stand at that row)
  auto walk_rows = [&](int first_row) __attribute__((always_inline)) {
  if constexpr (NBUF >= 2) {
    // Ring of NBUF row buffers: the loads run NBUF-1 rows ahead of the compute, which
    // hides the memory latency behind several rows of work.  Row q lives in buffer
    // q % NBUF; the buffer that row q + NBUF - 1 goes to was last read for row q - 1,
    // which every wave finished before the barrier that ended that row.
    constexpr int P = NBUF - 1;
#pragma unroll
    for (int u = 0; u < P; ++u) issue_row(u);
    RowMeta meta = load_meta();
    sync_rows(std::integral_constant<int, P - 1>{});  // row 0 has landed
    for (int r = first_row; r < nrows; r += NBUF) {
#pragma unroll
      for (int u = 0; u < NBUF; ++u) {
        if (r + u < nrows) {
          issue_row((u + P) % NBUF);
          const RowMeta next = load_meta();
          if (wave_live != 0) compute_row(u, meta);
          sync_rows(std::integral_constant<int, P - 1>{});  // the next row has landed
          meta = next;
        }
      }
    }
  } else {
    // one stage only (two do not fit in LDS): load, then compute
    for (int ir = first_row; ir < nrows; ++ir) {
      issue_row(0);
      const RowMeta meta = load_meta();
      sync_rows(std::integral_constant<int, 0>{});
      if (wave_live != 0) compute_row(0, meta);
      sync_rows(std::integral_constant<int, 0>{});
    }
  }
  };
  // Waves that own two key tiles (16-bit types, d <= 32) walk the plain rows at the start of
  // the chunk (not flagged, no masked key in any of the block's key tiles: the common case)
  // software-pipelined: a wave's matrix instructions of one tile are issued between the
  // exponentials and multiply-adds of the tile before it (the second tile of a row overlaps
  // the first, the first tile of the next row overlaps the second), so neither pipe waits
  // for the other although only one or two waves share a SIMD.  The next row's operands are
  // read from LDS a whole row ahead.  From the first row that is not plain on (padding: the
  // rows past the valid length) the loop above takes over.  (The same walk with the masked
  // form of the score needs about 290 registers per lane: it does not fit 8 waves.)
  constexpr bool kPipelined = WJ == 1 && WK == 2 && NBUF == 4 && sizeof(T) == 2 && D <= 32;
  if constexpr (kPipelined) {
    // the first row that is not plain: every thread looks at its share of the rows, the
    // smallest index wins (through a word of LDS, which is not yet in use)
    uint32_t* first_word = reinterpret_cast<uint32_t*>(tri_smem);
    if (tid == 0) *first_word = (uint32_t)nrows;
    __syncthreads();
    {
      const int w0 = k_blk / 32;
      for (int ir = tid; ir < nrows; ir += NW * 64) {
        bool ok = a.rowflag[(int64_t)b * N + i_begin + ir] == 0;
        const uint32_t* kw = a.keep + ((int64_t)b * N + i_begin + ir) * a.nwords;
#pragma unroll
        for (int w = 0; w < BKB / 32; ++w) ok = ok && (w0 + w < a.nwords ? kw[w0 + w] : 0u) == 0xffffffffu;
        if (!ok) {
          atomicMin(first_word, (uint32_t)ir);
          break;
        }
      }
    }
    __syncthreads();
    int nplain = __builtin_amdgcn_readfirstlane((int)*first_word);
    __syncthreads();
    if (nplain < 2 * NBUF) nplain = 0;  // too few to fill the pipeline
    if (nplain > 0) {
      struct RowOps {
        frag q[WJ][DS], dout[WJ][DS], k[WK][DS], v[WK][DS];
        frag df[WJ];    // -delta of the lane's query as a rank-1 operand
        float nl2[WJ];  // -lse of the lane's query in the exponent's unit
        uint32_t lw[WJ], dw[WJ];
      };
      auto read_ops = [&](int buf, RowOps& o) __attribute__((always_inline)) {
        const bool high = kHighSet && buf >= 2;
        const int sl = buf * STAGE - (high ? HIGH : 0);
        const OperandOffsets<T, D>& oq = high ? ofq_hi : ofq;
        const OperandOffsets<T, D>& ok = high ? ofk_hi : ofk;
        const int soff = high ? scalar_off_hi : scalar_off;
#pragma unroll
        for (int tj = 0; tj < WJ; ++tj) {
#pragma unroll
          for (int s = 0; s < DS; ++s) {
            o.q[tj][s] = oq.natural_at(sl + OFF_Q + tj * 32 * ROWB, s);
            o.dout[tj][s] = oq.natural_at(sl + OFF_DO + tj * 32 * ROWB, s);
          }
          o.lw[tj] = *reinterpret_cast<TRI_L3 const uint32_t*>((uintptr_t)(uint32_t)(sl + OFF_LSE + tj * 128 + soff));
          o.dw[tj] = *reinterpret_cast<TRI_L3 const uint32_t*>((uintptr_t)(uint32_t)(sl + OFF_DELTA + tj * 128 + soff));
        }
#pragma unroll
        for (int tk = 0; tk < WK; ++tk)
#pragma unroll
          for (int s = 0; s < DS; ++s) {
            o.k[tk][s] = ok.natural_at(sl + OFF_K + tk * 32 * ROWB, s);
            o.v[tk][s] = ok.natural_at(sl + OFF_V + tk * 32 * ROWB, s);
          }
      };
      auto finish_ops = [&](RowOps& o) __attribute__((always_inline)) {
#pragma unroll
        for (int tj = 0; tj < WJ; ++tj) {
          o.nl2[tj] = split_value<T>(o.lw[tj]) * c;
          o.df[tj] = drank[tj].set(g ? 0u : o.dw[tj]);
        }
      };
      // The tiles of a wave in the order they are walked: tile t is (t / WK, t % WK).  The
      // matrix instructions of tile TN of row `on` (scores from the bias tile, dP from
      // -delta) go into sn / dpn, dealt between the elementwise work of tile TC of row
      // `oc`, whose scores s and dP are complete: db += exp2(c s - lse) dP.
      constexpr int NT = WJ * WK;
      constexpr int NM = 2 * DS + 1;  // matrix instructions of a tile
      static_assert(NT % 2 == 0, "the two accumulator sets swap once per tile");
      auto phase = [&](const RowOps& on, auto tn_tag, f32x16& sn, f32x16& dpn, const RowOps& oc, auto tc_tag, const f32x16& s,
                       const f32x16& dp, auto&& between) __attribute__((always_inline)) {
        constexpr int TN = decltype(tn_tag)::value, TC = decltype(tc_tag)::value;
        constexpr int nj = TN / WK, nk = TN % WK, cj = TC / WK, ck = TC % WK;
        static_for<NM>([&](auto xc) __attribute__((always_inline)) {
          constexpr int X = decltype(xc)::value;
          // the two chains alternate, so that an instruction seldom waits for the one before it
          constexpr bool IS_S = X == 0 || (X >= 2 && X % 2 == 0 && X / 2 < DS);
          constexpr int before = (X - 1) / 2 < DS - 1 ? (X - 1) / 2 : DS - 1;  // score steps among slots 1 .. X-1
          constexpr int DI = X - 2 - before;                                    // dP steps among them, less the -delta one
          if constexpr (X == 0) sn = E::mfma(on.k[nk][0], on.q[nj][0], biasr[nj][nk]);
          else if constexpr (X == 1) dpn = E::mfma(ones, on.df[nj], zero16());
          else if constexpr (IS_S) sn = E::mfma(on.k[nk][X / 2], on.q[nj][X / 2], sn);
          else dpn = E::mfma(on.v[nk][DI], on.dout[nj][DI], dpn);
          between(std::integral_constant<int, TC * NM + X>{});
#pragma unroll
          for (int v = 16 * X / NM; v < 16 * (X + 1) / NM; ++v) {
            const float p = fast_exp2(__builtin_fmaf(s[v], c, oc.nl2[cj]));
            dbacc[cj][ck][v] = __builtin_fmaf(p, dp[v], dbacc[cj][ck][v]);
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      };
      constexpr int AHEAD = NBUF;  // rows between the loads and the compute
#pragma unroll
      for (int u = 0; u < AHEAD; ++u) issue_row(u);
      sync_rows(std::integral_constant<int, AHEAD - 2>{});  // rows 0 and 1 have landed
      // (two sets of operand registers that swap roles from row to row: no copies)
      RowOps ops[2];
      f32x16 sc[2], dpc[2];  // scores and dP of the tile in flight and the tile being consumed
      read_ops(0, ops[0]);
      finish_ops(ops[0]);
      // (the first tile of the first row has nothing to overlap with)
      sc[0] = E::mfma(ops[0].k[0][0], ops[0].q[0][0], biasr[0][0]);
#pragma unroll
      for (int sd = 1; sd < DS; ++sd) sc[0] = E::mfma(ops[0].k[0][sd], ops[0].q[0][sd], sc[0]);
      dpc[0] = E::mfma(ones, ops[0].df[0], zero16());
#pragma unroll
      for (int sd = 0; sd < DS; ++sd) dpc[0] = E::mfma(ops[0].v[0][sd], ops[0].dout[0][sd], dpc[0]);
      sc[1] = zero16();
      dpc[1] = zero16();
      sync_rows(std::integral_constant<int, AHEAD - 2>{});  // every wave has read row 0: its buffer is free
#ifdef TRI_DB_TIMING
      uint64_t t_wait = 0, t_barrier = 0;
      const uint64_t t_clk0 = __builtin_amdgcn_s_memtime(), t_real0 = __builtin_amdgcn_s_memrealtime();
#endif
      for (int r = 0; r < nplain; r += NBUF) {
#pragma unroll
        for (int u = 0; u < NBUF; ++u) {
          if (r + u < nplain) {
            RowOps& cur = ops[u & 1];
            RowOps& next = ops[(u + 1) & 1];
            // row r + u + NBUF goes into the buffer whose row is in registers already; its
            // loads are dealt over the row (a burst of them would hold up the wave's other
            // instructions until the memory pipeline has taken them all)
            const int64_t advance = next_row_advance();
            auto deal_loads = [&](auto slot_tag) __attribute__((always_inline)) {
              constexpr int slot = decltype(slot_tag)::value;
              static_for<XN>([&](auto xt) __attribute__((always_inline)) {
                constexpr int x = decltype(xt)::value;
#if !defined(TRI_DB_TIMING) || TRI_DB_TIMING_LOADS != 0
                if constexpr (slot == (x * NT * NM) / XN) issue_item(u, xt, advance);
#endif
              });
            };
            read_ops((u + 1) % NBUF, next);
            __builtin_amdgcn_sched_barrier(0);
            static_for<NT - 1>([&](auto tc) __attribute__((always_inline)) {
              constexpr int t = decltype(tc)::value;
              phase(cur, std::integral_constant<int, t + 1>{}, sc[(t + 1) & 1], dpc[(t + 1) & 1], cur, tc, sc[t & 1], dpc[t & 1], deal_loads);
            });
            finish_ops(next);
            phase(next, std::integral_constant<int, 0>{}, sc[0], dpc[0], cur, std::integral_constant<int, NT - 1>{}, sc[(NT - 1) & 1], dpc[(NT - 1) & 1], deal_loads);
#ifdef TRI_DB_TIMING
            {
              const uint64_t m0 = __builtin_amdgcn_s_memtime();
              asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" : : "n"((AHEAD - 2) * XN) : "memory");
              const uint64_t m1 = __builtin_amdgcn_s_memtime();
              asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
              const uint64_t m2 = __builtin_amdgcn_s_memtime();
              asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
              t_wait += m1 - m0;
              t_barrier += m2 - m1;
            }
#else
            sync_rows(std::integral_constant<int, AHEAD - 2>{});  // rows up to r + u + 2 have landed
#endif
          }
        }
      }
#ifdef TRI_DB_TIMING
      {
        const uint64_t t_clk1 = __builtin_amdgcn_s_memtime(), t_real1 = __builtin_amdgcn_s_memrealtime();
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        if (lane == 0) {
          uint64_t* rec = reinterpret_cast<uint64_t*>(a.db) + ((int64_t)L * NW + wave) * 4;
          rec[0] = t_clk1 - t_clk0;
          rec[1] = t_wait;
          rec[2] = t_barrier;
          rec[3] = t_real1 - t_real0;
        }
        return;
      }
#endif
      if (nplain < nrows) {
        // hand over: nothing in flight, the loads and the row words moved to row nplain
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const int at = min(rows_issued, nrows - 1);  // the row the loads stand at
#pragma unroll
        for (int x = 0; x < XN; ++x) item_base[x] += (int64_t)(nplain - at) * item_step[x];
        rows_issued = nplain;
        flag_word = (const_words)((uintptr_t)flag_word + (uintptr_t)((int64_t)nplain * 4));
        keep_word = (const_words)((uintptr_t)keep_word + (uintptr_t)((int64_t)nplain * keep_step));
        meta_rows = nplain;
      }
    }
    if (nplain < nrows) walk_rows(nplain);
  } else {
    walk_rows(0);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the spare rows loaded past the end
  if (wave_live == 0) return;

  // a single chunk writes db itself; several chunks write fp32 partials.  The lane
  // owns query j; its 16 values are two runs of 8 consecutive keys.
  const bool direct = a.nchunks == 1;
  T* db_bh = reinterpret_cast<T*>(a.db) + b * a.sdb_b + h * a.sdb_h;
  float* part = a.dbpart + ((int64_t)chunk * a.BH + bh) * N * N;
  const bool vec_store = (N % 8) == 0;
  // 16-byte stores of 8 keys need db contiguous along k with rows that stay aligned
  const bool db_vec = a.sdb_k == 1 && ((a.sdb_j | a.sdb_h | a.sdb_b) % 8) == 0;
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj) {
    const int j = j_wave + 32 * tj + jl;
    if (j >= N) continue;
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int key0 = k_wave + 32 * tk + 16 * r + 8 * g;
        if (!direct) {
          float* dst = part + (int64_t)j * N + key0;
          if (vec_store && key0 + 8 <= N) {
#pragma unroll
            for (int e4 = 0; e4 < 2; ++e4) {
              f32x4 ov;
#pragma unroll
              for (int e = 0; e < 4; ++e) ov[e] = dbacc[tj][tk][8 * r + 4 * e4 + e];
              *reinterpret_cast<f32x4*>(dst + 4 * e4) = ov;
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (key0 + e < N) dst[e] = dbacc[tj][tk][8 * r + e];
          }
          continue;
        }
        T* dst = db_bh + j * a.sdb_j + key0 * a.sdb_k;
        if (db_vec && key0 + 8 <= N) {
          if constexpr (sizeof(T) == 2) {
            typename E::vec ov;
#pragma unroll
            for (int e = 0; e < 8; ++e) ov[e] = (T)dbacc[tj][tk][8 * r + e];
            *reinterpret_cast<typename E::vec*>(dst) = ov;
          } else {
#pragma unroll
            for (int e4 = 0; e4 < 2; ++e4) {
              f32x4 ov;
#pragma unroll
              for (int e = 0; e < 4; ++e) ov[e] = dbacc[tj][tk][8 * r + 4 * e4 + e];
              *reinterpret_cast<f32x4*>(dst + 4 * e4) = ov;
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key0 + e < N) dst[e * a.sdb_k] = (T)dbacc[tj][tk][8 * r + e];
        }
      }
    }
  }
}

// db = sum over chunks of the fp32 partials, in chunk order
template <typename T>
__global__ __launch_bounds__(256) void tri_bwd_b_reduce_kernel(const BwdArgs a, int64_t count) {
  const int64_t x = (int64_t)blockIdx.x * 256 + threadIdx.x;  // ((bh * N) + j) * N + k
  if (x >= count) return;
  float acc = a.dbpart[x];
  for (int ch = 1; ch < a.nchunks; ++ch) acc += a.dbpart[(int64_t)ch * count + x];
  const int k = (int)(x % a.N), j = (int)((x / a.N) % a.N), bh = (int)(x / ((int64_t)a.N * a.N));
  reinterpret_cast<T*>(a.db)[(bh / a.H) * a.sdb_b + (bh % a.H) * a.sdb_h + j * a.sdb_j + k * a.sdb_k] = (T)acc;
}

}  // namespace tri
