// Row-resident backward: dq, dk and dv of one pair row from ONE computation of the
// scores and of dP (the dq kernel and the dk/dv kernel each recompute both).
//
// Work unit: (batch*head, pair row i), one workgroup of four waves, one wave per
// SIMD with the whole register file.  The keys of the row are dealt to the waves
// in tiles of 32 (wave w owns key tiles w, w+4, ...; at most KT of them): their
// dk, dv accumulators stay in registers for the whole row, their V rows too (B
// operands; in a private piece of LDS where the registers do not hold them all), and
// the K row of the pair row sits in LDS for the whole workgroup (read as B operand of
// the scores and, transposed, as A operand of dq).  The queries of the row are
// streamed through LDS in tiles of 32 (Q, dO rows, direct global->LDS loads, three
// stages: in use, ready, in flight).  Per (query tile, key tile), with the scores
// un-transposed (a lane owns one key and 16 queries):
//   S  = Q K^T + sqrt(d) (bias - lse)      every term through the matrix pipe (below)
//   P  = exp2(c S)
//   dP = dO V^T - delta
//   dS = P * dP
//   dv^T += dO^T P,  dk^T += Q^T dS        P, dS are B operands as they are
//   dq^T += K^T dS^T                       dS goes through a 2 KiB LDS tile of the wave
//                                          and comes back transposed (ds_read_tr)
// Everything additive is a matrix product, which leaves the per-tile vector work free of
// conversions, selects and adds (matrix and full-rate vector time add up within a wave,
// so this costs what it saves for the bias; it makes masked rows cost what unmasked ones
// do and frees the registers the converted tiles took).  The packed bias words of a tile are A operands as they
// are (a lane owns a query and eight keys) against a constant B operand that holds
// sqrt(d) where the contraction slot is the column's key; -lse sqrt(d) and -delta (per
// query) and the key mask (per key) are rank-1 products of operand words.  That leaves
// the vector ALU one multiply and one exp2 per score, one multiply per dS and the two
// conversions.  dq of a query tile is the sum of the four waves' partial tiles: they
// meet in LDS once per query tile (one barrier) and each wave adds a quarter of the tile, its
// own part first and then the others' in wave order (deterministic, no atomics), behind the
// MFMAs that start the next query tile.
// The four waves share the LDS pipe, and an LDS instruction occupies it for four cycles
// whatever its width (transposing reads move half of what 16-byte reads do): operands
// that do not change over the key tiles of a query tile (Q^T, dO^T) are read once per
// query tile where the registers allow.
//
// The prologue also computes delta = rowsum(o * do) of the row and leaves it, with
// the row's log-sum-exp, in the per-query planes the db kernel reads.
//
// Rows up to 128*KT keys fit (1024 keys at head dim 32).  Longer rows run the kernel in
// several passes (MULTI), one launch per 128*KT keys: dk and dv of a pass's keys are complete
// after it, dq is the sum over the passes and travels from one to the next as two numbers of
// the element type per value (the rounded running sum in dq itself, the rounding error in a
// workspace plane), which keeps 16 bits of it.  The per-query words are then read from the
// global planes (the first pass writes them) instead of LDS, where the longer row leaves
// them no room.  Replaces _bwd_q and _bwd_kv of reference
// src/trifast/triton.py:274-383 and :143-263 in one pass.
#pragma once
#include <type_traits>
#include <utility>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

// -DTRI_ROW_TIMING builds the kernel as a probe of itself (benchmark/microbench/row_timeline.py):
// wave 0 of every workgroup reads the 100 MHz counter at the marks below and the shader clock
// between the steps of the query-tile loop, and leaves the readings where the db argument
// points (a buffer of the caller's; db itself is not computed by this kernel).
#ifdef TRI_ROW_TIMING
#define TRI_ROW_MARK(var)               \
  __builtin_amdgcn_sched_barrier(0);    \
  const uint64_t var = __builtin_amdgcn_s_memrealtime(); \
  __builtin_amdgcn_sched_barrier(0)
#define TRI_ROW_TICK(k)                                      \
  do {                                                       \
    __builtin_amdgcn_sched_barrier(0);                       \
    const uint64_t now_ = __builtin_amdgcn_s_memtime();      \
    tacc[k] += now_ - tprev;                                 \
    tprev = now_;                                            \
    __builtin_amdgcn_sched_barrier(0);                       \
  } while (0)
#else
#define TRI_ROW_MARK(var) (void)0
#define TRI_ROW_TICK(k) (void)0
#endif

namespace tri {

constexpr int kRowWaves = 4;

// ---- the MFMA order of one step of the kernel below ------------------------------------
enum RowOp { R_SOFF, R_SB, R_SQK, R_DOFF, R_DP, R_ACC, R_DQ };
struct RowSched {
  int n;             // MFMAs of the step
  int kind[48], idx[48];
  int dq_reads_at;   // the LDS reads for dq follow this MFMA
  int last_sqk;      // the last MFMA that reads the K rows of the next tile
  int v_reads_at;    // V operands kept in LDS are read after this MFMA
  int last_sb;       // the last MFMA that reads bias words (0 without any)
};
// Two dependent chains start a tile (scores: per-query offset and key mask, bias parts,
// q.k; dP: -delta, dO.v) and three finish the one before (dv/dk, dq).  Dependent MFMAs are
// kept apart: first the head of the score chain alternates with the dv/dk MFMAs, then dq,
// the q.k part and the dP chain take turns.
constexpr RowSched make_row_sched(bool has_prev, bool has_next, bool flagged, int nsb, int ds, int nacc, int ndq) {
  RowSched s{};
  s.dq_reads_at = -1;
  s.last_sqk = -1;
  s.v_reads_at = -1;
  s.last_sb = 0;
  int lk[16] = {}, li[16] = {}, ns = 0;
  if (has_next) {
    lk[ns] = R_SOFF;
    li[ns++] = 0;
    if (!flagged)
      for (int i = 0; i < nsb; ++i) {
        lk[ns] = R_SB;
        li[ns++] = i;
      }
  }
  const int na = has_prev ? nacc : 0;
  int is = 0, ia = 0;
  if (is < ns) {
    if (lk[is] == R_SB) s.last_sb = s.n;
    s.kind[s.n] = lk[is];
    s.idx[s.n++] = li[is++];
  }
  while (is < ns || ia < na) {
    if (is < ns) {
      if (lk[is] == R_SB) s.last_sb = s.n;
      s.kind[s.n] = lk[is];
      s.idx[s.n++] = li[is++];
    }
    if (ia < na) {
      s.kind[s.n] = R_ACC;
      s.idx[s.n++] = ia++;
    }
  }
  const int nq = has_prev ? ndq : 0, nk = (has_next && !flagged) ? ds : 0, np = has_next ? 1 + ds : 0;
  int iq = 0, ik = 0, ip = 0, first_dq = -1;
  while (iq < nq || ik < nk || ip < np) {
    if (iq < nq) {
      if (first_dq < 0) first_dq = s.n;
      s.kind[s.n] = R_DQ;
      s.idx[s.n++] = iq++;
    }
    if (ik < nk) {
      s.last_sqk = s.n;
      s.kind[s.n] = R_SQK;
      s.idx[s.n++] = ik++;
    }
    if (ip < np) {
      if (ip == 1) s.v_reads_at = s.n >= 4 ? s.n - 4 : 0;
      s.kind[s.n] = ip == 0 ? R_DOFF : R_DP;
      s.idx[s.n++] = ip == 0 ? 0 : ip - 1;
      ++ip;
    }
  }
  if (first_dq >= 0) s.dq_reads_at = first_dq >= 3 ? first_dq - 3 : 0;
  return s;
}
template <bool HAS_PREV, bool HAS_NEXT, bool FLAGGED, int NSB, int DS, int NACC, int NDQ>
struct RowSchedOf {
  static constexpr RowSched value = make_row_sched(HAS_PREV, HAS_NEXT, FLAGGED, NSB, DS, NACC, NDQ);
};

// Key tiles per wave whose V operands live in LDS instead of registers: the longest rows
// leave the vector registers no room for all of them (the accumulators fill the other file).
// (one tile more in LDS when the row takes several passes: the words of the queries then leave
// LDS the room, and the dq carried between the passes takes registers)
constexpr int bwd_row_v_lds_tiles(int D, int KT, bool multi = false) { return KT * (D / 16) < 16 ? 0 : D <= 32 ? KT - (multi ? 2 : 3) : 1; }
// LDS bytes of the kernel below.  dq partials: two buffers (one barrier per query tile) of
// three quarters of a tile per wave (the quarter a wave sums itself waits in its dS tile)
constexpr int bwd_row_red_bytes(int D) { return kRowWaves * 3 * ((D + 31) / 32) * 1024; }
constexpr int bwd_row_base_lds_bytes(int D, int es, int KT, bool multi) {  // (without the per-query words)
  const int rowb = D * es, keys = kRowWaves * KT * 32;
  return keys * rowb + 3 * (2 * 32 * rowb) + kRowWaves * 2048 + 2 * bwd_row_red_bytes(D) +
         kRowWaves * bwd_row_v_lds_tiles(D, KT, multi) * (D / 16) * 1024;
}
// The per-query operand words of the row (two planes of 4 bytes per query) live in LDS where
// there is room and the row takes one pass; else they come from the global planes that the
// prologue writes, one query tile ahead.
constexpr bool bwd_row_words_in_lds(int D, int es, int KT, bool multi) {
  return !multi && bwd_row_base_lds_bytes(D, es, KT, multi) + 2 * kRowWaves * KT * 32 * 4 <= 160 * 1024;
}
constexpr int bwd_row_lds_bytes(int D, int es, int KT, bool multi = false) {
  return bwd_row_base_lds_bytes(D, es, KT, multi) + (bwd_row_words_in_lds(D, es, KT, multi) ? 2 * kRowWaves * KT * 32 * 4 : 0);
}

template <typename T, int D, int KT, bool MULTI = false>
__global__ __launch_bounds__(kRowWaves * 64, 1) void tri_bwd_row_kernel(const BwdArgs a) {
  static_assert(sizeof(T) == 2, "16-bit inputs only (the transposing LDS reads)");
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  using DsTile = LdsTile<T, 32, 2>;  // the wave's dS tile: 16-byte stores of whole rows, transposed reads
  constexpr int NWV = kRowWaves;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 2;
  constexpr int ROWB = Tile::ROWB;
  constexpr int KEYS = NWV * KT * 32;         // keys (and queries) the workgroup can hold
  constexpr bool WORDS_LDS = bwd_row_words_in_lds(D, (int)sizeof(T), KT, MULTI);  // per-query words of the row in LDS (else from the global planes)
  constexpr int STAGE = 2 * 32 * ROWB;        // Q tile | dO tile
  constexpr int OFF_K = 0;
  constexpr int OFF_ST = KEYS * ROWB;
  constexpr int OFF_DS = OFF_ST + 3 * STAGE;  // three stages: in use, ready, in flight
  constexpr int OFF_RED = OFF_DS + NWV * 2048;
  constexpr int OFF_NL = OFF_RED + 2 * bwd_row_red_bytes(D);
  constexpr int PLANE = WORDS_LDS ? KEYS * 4 : 0;  // per-query words of the row
  constexpr int OFF_ND = OFF_NL + PLANE;
  constexpr int G2W = (2 * 32 * (ROWB / 16) / 64 + NWV - 1) / NWV;  // global->LDS loads per wave and stage
  constexpr int VL = bwd_row_v_lds_tiles(D, KT, MULTI);  // this wave's last VL key tiles keep V in LDS
  constexpr int VR = KT - VL;
  constexpr int OFF_V = OFF_ND + PLANE;
  static_assert(OFF_V + NWV * VL * DS * 1024 == bwd_row_lds_bytes(D, (int)sizeof(T), KT, MULTI), "the launcher sizes LDS with bwd_row_lds_bytes");
  static_assert(bwd_row_lds_bytes(D, (int)sizeof(T), KT, MULTI) <= 160 * 1024, "LDS of one compute unit");
  static_assert((KT - 1) * NWV * 32 * ROWB + 32 * ROWB <= 65536, "key tile offsets are LDS immediates");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  TRI_ROW_MARK(t_entry);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kl = lane & 31, g = lane >> 5;
  const int N = a.N;
  const int NJ = a.nwords;  // 32-tiles of the row (queries and keys)
  // this pass: key tiles KT0 .. KT0 + 4 KT - 1 of the row (tiles past the row's end are empty)
  const int KT0 = MULTI ? a.key_tile0 : 0;
  const bool first_pass = !MULTI || (a.pass_flags & 1) == 0, last_pass = !MULTI || (a.pass_flags & 2) == 0;

  // Workgroups go to the 8 XCDs round-robin by linear id.  Every XCD walks its own
  // contiguous run of (batch*head, row) items, so that at any time it works on one
  // head (or two) and that head's packed bias stays in its L2.
  const int total = a.BH * N;
  const int per_xcd = (total + 7) / 8;
  const int L = blockIdx.x;
  const int item = (L & 7) * per_xcd + (L >> 3);
  if ((L >> 3) >= per_xcd || item >= total) return;
  const int bh = item / N, i = item % N;
  const int b = bh / a.H, h = bh % a.H;

  const T* qrow = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h + i * a.sq.i;
  const T* krow = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h + i * a.sk.i;
  const T* vrow = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h + i * a.sv.i;
  const T* dorow = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h + i * a.sdo.i;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;

  unsigned char* const lds_k = tri_smem + OFF_K;
  uint32_t* const nl = reinterpret_cast<uint32_t*>(tri_smem + OFF_NL);  // operand words, see split_word
  uint32_t* const nd = reinterpret_cast<uint32_t*>(tri_smem + OFF_ND);

  // ---- prologue -----------------------------------------------------------------
  // K row -> LDS (rows past the end repeat the last key; their keep bits are clear)
  Tile::template fill<KEYS, NWV>(lds_k, [&](int r) { return krow + (int64_t)min(32 * KT0 + r, N - 1) * a.sk.j; }, wave, lane);
  // query tiles 0 (and 1) -> the two stage buffers
  // (per-lane source pointers for query tile 0, computed once; a tile inside the row adds
  // one uniform offset, the ragged last one clamps the query index)
  // The loads are written as asm: the compiler makes every LDS read that follows a
  // global->LDS load it knows of wait for that load (the read might be of the bytes in
  // flight), which would turn the prefetch of the next query tile into a stall at the next
  // operand read.  Here the stage in flight is not read before the wait and barrier that end
  // the query tile.  The compiler's own waits stay correct: loads return in issue order, and
  // a load it does not know of only makes the counter it waits on larger.  (The source
  // addresses are rebuilt from the lane id every time: kept in registers from one query tile
  // to the next they would be spilled, and a reload from scratch waits for every load in flight.)
  auto issue_stage = [&](int jt, int buf) {
    unsigned char* st = tri_smem + OFF_ST + buf * STAGE;
    int lane_now = lane;
    asm volatile("" : "+v"(lane_now));  // (opaque: nothing derived from it is hoisted out of the loop)
    // the stage is one 64-row tile (Q rows, then dO rows) of G2 wave loads of 1 KiB; every
    // wave issues the same number of them (with fewer loads than waves some are issued twice)
    constexpr int G2 = 2 * 32 * Tile::CPR / 64;
    const int jrow = 32 * jt;
#pragma unroll
    for (int x = 0; x < (G2 + NWV - 1) / NWV; ++x) {
      const int gi = (x * NWV + wave) % G2;
      const bool is_q = gi < G2 / 2;  // wave-uniform
      const T* rows = is_q ? qrow : dorow;
      const int64_t stride = is_q ? a.sq.j : a.sdo.j;
      const int p = gi * 64 + lane_now;
      const int r = p / Tile::CPR, cc = (p % Tile::CPR) ^ Tile::swz(r);
      // a 64-bit base per tile (scalar registers) and a 32-bit byte offset per lane; rows past
      // the end of the pair row (last tile only) read the last row again
      const T* base = rows + (int64_t)jrow * stride;
      const uint32_t voff = (uint32_t)(min(r & 31, N - 1 - jrow) * (int)stride + cc * Tile::VEC) * (uint32_t)sizeof(T);
      const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(TRI_L3 unsigned char*)(st + gi * 1024));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(voff), "s"(base) : "memory", "m0");
    }
  };
  issue_stage(0, 0);
  issue_stage(min(1, NJ - 1), 1);

  // a fully masked row drops q.k and the bias from its scores (all logits equal)
  // (these words come through the scalar cache, all in flight together and apart from the
  // vector loads around them)
  const bool flagged = uniform_word(a.rowflag, b * N + i) != 0;
  // keep words of this wave's key tiles (bit k set = key k of the tile is attended)
  uint32_t kw[KT];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int kt = KT0 + NWV * t + wave;
    kw[t] = uniform_word(a.keep, (b * N + i) * a.nwords + min(kt, NJ - 1));
  }
#pragma unroll
  for (int t = 0; t < KT; ++t)
    if (KT0 + NWV * t + wave >= NJ) kw[t] = 0u;
  TRI_ROW_MARK(t_p1);
  const uint32_t lanebit = 1u << kl;

  // V rows of this lane's keys as B operands: in registers for the wave's first VR key
  // tiles, in a private piece of LDS (operand by operand, 16 bytes per lane) for the rest
  frag vf[VR > 0 ? VR : 1][DS];
  frag* const v_lds = reinterpret_cast<frag*>(tri_smem + OFF_V + wave * VL * DS * 1024) + lane;
  // (every load of the prologue is issued before the first one is used: the V rows here, then
  // the row's o and do for delta (queries past the end read the last one again): one trip to
  // memory for all of them, while the K row is on its way to LDS)
  frag vx[KT][DS];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int key = min(32 * (KT0 + NWV * t + wave) + kl, N - 1);
#pragma unroll
    for (int s = 0; s < DS; ++s) vx[t][s] = *reinterpret_cast<const frag*>(vrow + (int64_t)key * a.sv.j + 2 * KP * s + KP * g);
  }
  const T* const orow = reinterpret_cast<const T*>(a.o) + ((int64_t)bh * N + i) * N * D;
  const float* const lserow = a.lse + ((int64_t)bh * N + i) * N;
  constexpr int NIT = WORDS_LDS ? (KEYS + NWV * 64 - 1) / (NWV * 64) : 1;  // queries per thread (single pass)
  typename E::vec ov[NIT][D / 8], dv[NIT][D / 8];
  float lv[NIT];
  if constexpr (WORDS_LDS) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int jc = min(tid + it * NWV * 64, N - 1);
#pragma unroll
      for (int s = 0; s < D / 8; ++s) {
        ov[it][s] = *reinterpret_cast<const typename E::vec*>(orow + (int64_t)jc * D + 8 * s);
        dv[it][s] = *reinterpret_cast<const typename E::vec*>(dorow + (int64_t)jc * a.sdo.j + 8 * s);
      }
      lv[it] = lserow[jc];
    }
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int t = 0; t < KT; ++t)
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      if (t < VR) vf[t][s] = vx[t][s];
      else v_lds[((t - VR) * DS + s) * 64] = vx[t][s];
    }

  TRI_ROW_MARK(t_p2);
  // per-query terms of the row: -delta and -lse*sqrt(d) (ln n for lse in a fully masked
  // row) as MFMA operand words, kept in LDS for this kernel and written for the db kernel
  uint32_t* const dplane = a.delta + ((int64_t)bh * N + i) * N;
  uint32_t* const lplane = a.lse2 + ((int64_t)bh * N + i) * N;
  if (first_pass) {
    const float flat = -__builtin_amdgcn_logf((float)N) * (kLn2 * a.sqrt_d);
    auto query_words = [&](int j, float dsum, float lse_j) {
      float nlv = E::kMaskElem, ndv = 0.f;  // queries past the end: P = dS = 0
      if (j < N) {
        ndv = -dsum;
        nlv = flagged ? flat : -lse_j * a.sqrt_d;
      }
      const uint32_t lw = split_word<T>(nlv), dw = split_word<T>(ndv);
      if (j < N) {
        dplane[j] = dw;
        lplane[j] = lw;
      }
      if constexpr (WORDS_LDS) {
        nl[j] = lw;
        nd[j] = dw;
      }
    };
    if constexpr (WORDS_LDS) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int j = tid + it * NWV * 64;
        float dsum = 0.f;
#pragma unroll
        for (int s = 0; s < D / 8; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) dsum += (float)ov[it][s][e] * (float)dv[it][s][e];
        if (KEYS % (NWV * 64) == 0 || j < KEYS) query_words(j, dsum, lv[it]);
      }
    } else {
      for (int j = tid; j < N; j += NWV * 64) {
        float dsum = 0.f;
#pragma unroll
        for (int s = 0; s < D / 8; ++s) {
          const typename E::vec ov = *reinterpret_cast<const typename E::vec*>(orow + (int64_t)j * D + 8 * s);
          const typename E::vec dv = *reinterpret_cast<const typename E::vec*>(dorow + (int64_t)j * a.sdo.j + 8 * s);
#pragma unroll
          for (int e = 0; e < 8; ++e) dsum += (float)ov[e] * (float)dv[e];
        }
        query_words(j, dsum, lserow[j]);
      }
    }
  }
  TRI_ROW_MARK(t_p3);
  // (words not in LDS: they come back from the global planes, which the first pass has just
  // written: its stores are waited for, with the loads, before the barrier below; the loads
  // are made at device scope so that no stale copy in the first-level cache can serve them)
  auto fetch_words = [&](int jt, uint32_t& lw, uint32_t& dw) {
    const int j = 32 * min(jt, NJ - 1) + perm32(kl);
    lw = split_word<T>(E::kMaskElem);  // queries past the end: P = dS = 0
    dw = split_word<T>(0.f);
    if (j < N) {
      lw = __hip_atomic_load(lplane + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      dw = __hip_atomic_load(dplane + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };

  // lane-constant LDS offsets.  Q, dO tiles: natural A operands (tile row m stands for
  // query perm32(m)) and transposed A operands; K tiles: natural B operand of this lane's
  // key and transposed A operand; the wave's dS tile: write offsets and transposed reads.
  OperandOffsets<T, D> ofq, ofk;
  ofq.init(perm32(kl), lane);
  ofk.init(kl, lane);
  ofk.shift(wave * 32 * ROWB);  // key tile t of this wave starts (4 t + wave) * 32 rows into K
  OperandOffsets<T, 32, 2> ofd;
  ofd.init(0, lane);
  // (one tile: the wave reads dS of a key tile back before it writes the next one)
  unsigned char* const ds_tile = tri_smem + OFF_DS + wave * 2048;
  const int ds_w0 = DsTile::off(kl, 16 * g), ds_w1 = DsTile::off(kl, 32 + 16 * g);


  // packed bias tiles of this lane: tile (jt, kt) is 2 x 16 bytes per lane
  typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
  // (as A operand: operand row m stands for query perm32(m), like the Q and dO operands)
  // (a tile's address is a wave-uniform base, computed on the scalar unit, plus this lane's
  // constant 32-bit byte offset: no vector arithmetic per tile)
  uint32_t bias_lane = (uint32_t)((perm32(kl) + 32 * g) * 8 * sizeof(T));
  asm volatile("" : "+v"(bias_lane));
  auto bias_load = [&](int jt, int t, u32x4v* dst) {
    const int kt = min(KT0 + NWV * t + wave, a.NP - 1);
    const char* tile = reinterpret_cast<const char*>(pack_bh + ((int64_t)min(jt, a.NP - 1) * a.NP + kt) * 1024);
    uint32_t vo = bias_lane;
    asm volatile("" : "+v"(vo));  // (opaque here: the sum of the lane offset and the head's base is not hoisted as a 64-bit vector)
    dst[0] = *reinterpret_cast<const u32x4v*>(tile + (uint64_t)vo);
    dst[1] = *reinterpret_cast<const u32x4v*>(tile + (uint64_t)vo + 512 * sizeof(T));
  };
  const float c = a.c;

  // sqrt(d) * bias through the matrix pipe.  Half r of a packed bias tile gives a lane
  // (query, g) the keys 16 r + 8 g + 0..7 as its contraction slots; the constant B operand
  // of half r holds sqrt(d) in the slot that stands for the lane's own key (column) and
  // zero elsewhere.  sqrt(32) is not a 16-bit number: it goes in as hi + lo, one MFMA each.
  constexpr int NPART = D == 32 ? 2 : 1;
  constexpr int NSB = 2 * NPART;
  frag bsel[2][NPART];
  {
    const T hi = (T)a.sqrt_d;
    const T part[2] = {hi, (T)(a.sqrt_d - (float)hi)};
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int pp = 0; pp < NPART; ++pp) {
        const int e = kl - 16 * r - 8 * g;
        const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, part[pp]) << (16 * (e & 1));
        u32x4v w;
#pragma unroll
        for (int x = 0; x < 4; ++x) w[x] = (e >= 0 && e < 8 && (e >> 1) == x) ? bits : 0u;
        asm volatile("" : "+v"(w));  // resident: not rebuilt from the lane id at every use
        bsel[r][pp] = __builtin_bit_cast(frag, w);
      }
  }
  // rank-1 operands: per-query words (A side) and the ones / key-mask operand (B side)
  typename OffsetMask<T>::Queries s_off;
  s_off.init(0u, g);
  Rank1<T> d_off;
  d_off.init();
  typename OffsetMask<T>::Keys keys_op;
  keys_op.init(kl, g);

  // dq partial tiles of the four waves.  Wave q sums quarter q of every lane's values: head-dim
  // elements 32 mt + 8 q + 4 g + 0..3 of query 32 jt + kl, 8 bytes per lane (the four waves'
  // stores complete the rows).  The other three waves leave their parts of that quarter in
  // [buffer][summing wave q][slot][mt][lane] x 16 bytes, the slot being the writer's rank among
  // those three; the wave's own part waits in its dS tile, which is idle between the last key
  // tile of a query tile and the first of the next.  A wave adds its own part first, then the
  // others' in wave order (deterministic, no atomics).
  // The store is written as asm: a store the compiler knows of makes its waits for loads
  // waits for everything in flight (stores and loads retire out of order with each other).
  // Addresses are rebuilt from the lane id at every use: kept in registers across the
  // key-tile steps they would be spilled, and a reload from scratch waits for every load
  // in flight.
  static_assert(DM * 1024 <= 2048, "the own quarter of a dq tile fits the wave's dS tile");
  constexpr int RED_BYTES = bwd_row_red_bytes(D);
  // byte offsets in LDS, all wave-uniform and the same for every query tile: where this wave
  // leaves quarter q of its tile (per buffer), where its own quarter waits, and where the other
  // waves leave their parts of its quarter (three slots side by side)
  int part_wr[2][NWV];
#pragma unroll
  for (int q = 0; q < NWV; ++q)
#pragma unroll
    for (int bf = 0; bf < 2; ++bf)
      part_wr[bf][q] = q == wave ? OFF_DS + wave * 2048 : OFF_RED + bf * RED_BYTES + (q * 3 + (wave < q ? wave : wave - 1)) * DM * 1024;
  const int part_own = OFF_DS + wave * 2048, part_rd = OFF_RED + wave * 3 * DM * 1024;
  T* dqrow = reinterpret_cast<T*>(a.dq) + b * a.sdq.b + h * a.sdq.h + i * a.sdq.i;
  T* lorow = reinterpret_cast<T*>(a.dq_lo) + ((int64_t)bh * N + i) * N * D;  // (several passes only)
  typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
  // what the passes before this one left for this lane's elements of query tile jt: fetched at
  // the start of the query tile, added when its dq is summed
  struct DqCarry {
    typename E::vec4 hi[DM], lo[DM];
  };
  auto fetch_carry = [&](int jt, DqCarry& cy) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const int j = min(32 * jt + (ln & 31), N - 1);
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      const int d0 = min(32 * mt + 8 * wave + 4 * (ln >> 5), D - 4);
      cy.hi[mt] = *reinterpret_cast<const typename E::vec4*>(dqrow + (int64_t)j * a.sdq.j + d0);
      cy.lo[mt] = *reinterpret_cast<const typename E::vec4*>(lorow + (int64_t)j * D + d0);
    }
  };
  // this wave's dq tile of a query tile -> LDS, a quarter for each wave that sums one
  auto store_partials = [&](int buf, const f32x16 (&acc)[DM]) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int q = 0; q < NWV; ++q)
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        f32x4 x;
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[mt][4 * q + e];
        *(reinterpret_cast<f32x4*>(tri_smem + (buf ? part_wr[1][q] : part_wr[0][q]) + mt * 1024) + ln) = x;
      }
  };
  // the four parts of this wave's quarter: its own, then the other waves' in wave order
  struct DqParts {
    f32x4 v[NWV][DM];
  };
  auto load_partials = [&](int buf, DqParts& pp) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const f32x4* own = reinterpret_cast<const f32x4*>(tri_smem + part_own) + ln;
    const f32x4* others = reinterpret_cast<const f32x4*>(tri_smem + part_rd + (buf ? RED_BYTES : 0)) + ln;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      pp.v[0][mt] = own[mt * 64];
#pragma unroll
      for (int k = 0; k < 3; ++k) pp.v[1 + k][mt] = others[(k * DM + mt) * 64];
    }
  };
  // Their sum (the own part first, then the others in wave order), scaled, as the stores will write it: dq, what rounding it to the
  // element type lost (between the passes over a long row), and this lane's byte offset from
  // the start of the query tile in dq (~0: nothing to store).  The sum is cut into pieces of a
  // few instructions each (piece 0 .. kSumPieces-1, in this order): they run one per MFMA of a
  // step that has no vector work of its own, in the shadow of the matrix pipe.
  struct DqOut {
    f32x4 sum[DM];
    u32x2v hi[DM], lo[DM];
    uint32_t off;
  };
  constexpr int kSumPieces = 6;
  auto sum_dq_piece = [&](int piece, int jt, const DqParts& pp, const DqCarry& cy, DqOut& o) {
    if (piece == 0) {
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) o.sum[mt] = pp.v[0][mt] + pp.v[1][mt];
    } else if (piece == 1 || piece == 2) {
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) o.sum[mt] += pp.v[piece + 1][mt];
    } else if (piece == 3) {
#pragma unroll
      for (int mt = 0; mt < DM; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) o.sum[mt][e] *= a.scale;
      if constexpr (MULTI) {
        if (!first_pass) {
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) o.sum[mt][e] += (float)cy.hi[mt][e] + (float)cy.lo[mt][e];
        }
      }
    } else if (piece == 4) {
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        typename E::vec4 ov, lv;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ov[e] = (T)o.sum[mt][e];
          lv[e] = MULTI ? (T)(o.sum[mt][e] - (float)ov[e]) : (T)0.f;
        }
        o.hi[mt] = __builtin_bit_cast(u32x2v, ov);
        o.lo[mt] = __builtin_bit_cast(u32x2v, lv);
      }
    } else {
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int jl = ln & 31, d0 = 8 * wave + 4 * (ln >> 5);
      const bool live = jt >= 0 && jl < N - 32 * jt && d0 < D;
      // (row strides of the gradients are below 2^24 elements, like those of the inputs)
      o.off = live ? (__umul24((uint32_t)jl, (uint32_t)a.sdq.j) + (uint32_t)d0) * (uint32_t)sizeof(T) : ~0u;
    }
  };
  // (a 64-bit base per query tile in scalar registers and the 32-bit byte offset of the lane)
  auto store_dq = [&](int jt, const T* base, const DqOut& o) {
    const T* base_lo = lorow + (int64_t)(32 * jt) * D;
    if (o.off != ~0u) {
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        if (32 * mt + 8 * wave >= D) continue;  // (wave-uniform; head dims that are no multiple of 32)
        asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3" : : "v"(o.off), "v"(o.hi[mt]), "s"(base), "n"(64 * mt) : "memory");
        if constexpr (MULTI) {
          if (!last_pass) {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const uint32_t off_lo = (uint32_t)((ln & 31) * D + 8 * wave + 4 * (ln >> 5)) * (uint32_t)sizeof(T);
            asm volatile("global_store_dwordx2 %0, %1, %2 offset:%3" : : "v"(off_lo), "v"(o.lo[mt]), "s"(base_lo), "n"(64 * mt) : "memory");
          }
        }
      }
    }
  };

  TRI_ROW_MARK(t_p4);
  wait_dma_known();
  __syncthreads();

  // ---- query tiles ------------------------------------------------------------------
  // The loop exists in three versions, chosen once per wave: every key of the wave's
  // tiles attended (no mask work), some keys masked out, and a fully masked row (no q.k,
  // no bias).  Inside a query tile the key tiles run as a software pipeline: the score
  // and dP MFMAs of tile t+1 are issued before the exponentials of tile t, and the dq
  // MFMAs of tile t-1 (whose dS has been through LDS by then) after them.
  auto query_tiles = [&](auto masked_tag, auto flagged_tag) __attribute__((always_inline)) {
    constexpr bool FLAGGED = decltype(flagged_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value || FLAGGED;
    // (each version has its own accumulators, from zeroing to the final stores: merging
    // the versions' accumulators where they meet would copy all of them)
    f32x16 dkacc[KT][DM], dvacc[KT][DM];
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        E::mfma_acc_zero(dkacc[t][mt]);
        E::mfma_acc_zero(dvacc[t][mt]);
      }
    // The wave is alone on its SIMD, so nothing but its own instruction order hides a
    // latency: the code below is laid out as the schedule it should run in, and scheduling
    // barriers between the pieces keep the compiler from re-ordering it.
    auto SB = [] { __builtin_amdgcn_sched_barrier(0); };
    constexpr int NACC = 2 * PS * DM;  // dv, dk MFMAs of a tile
    constexpr int NDQ = PS * DM;       // dq MFMAs of a tile
    // packed bias of key tile t (t >= KT: tile t - KT of the next query tile) -> the ring slot
    // of that tile's parity, fetched two steps before its use (global memory, through L2).
    // (With an odd KT, tile 0 of the next query tile goes to the slot that tile KT-1 is read
    // from in the same step: its fetch follows the last MFMA that reads bias words.)
    u32x4v bias_ring[2][2] = {};
    auto fetch_bias = [&](int jt, int t) {
      if constexpr (!FLAGGED) bias_load(jt + t / KT, t % KT, bias_ring[(t % KT) % 2]);
    };
    fetch_bias(0, 0);
    fetch_bias(0, 1);
    uint32_t lw_next = 0u, dw_next = 0u;  // words from the global planes: those of the next query tile
    if constexpr (!WORDS_LDS) fetch_words(0, lw_next, dw_next);
    DqCarry carry;
    const T* dq_base = dqrow;  // dq of the query tile before the current one (from the second on)
    // dq of a query tile is summed over the waves, and stored, during the first step of the
    // next query tile, which has no vector work of its own.
    int buf = 0;  // jt % 3: the stage of this query tile
#ifdef TRI_ROW_TIMING
    uint64_t tacc[KT + 5] = {};  // shader clocks per step, summed over the query tiles
    const uint64_t t_clk0 = __builtin_amdgcn_s_memtime(), t_loop0 = __builtin_amdgcn_s_memrealtime();
    uint64_t tprev = t_clk0;
#endif
    for (int jt = 0; jt < NJ; ++jt) {
      const int buf_fill = buf == 0 ? 2 : buf - 1;  // (jt + 2) % 3: the stage to refill
      DqParts parts;  // (of the query tile before this one)
      DqOut dq_words;
      f32x16 dqacc[DM];  // (the first dq MFMA of a query tile starts it from zero)
      const unsigned char* qt = tri_smem + OFF_ST + buf * STAGE;
      const unsigned char* dot = qt + 32 * ROWB;

      // operand words of this lane's query (lanes 32..63 carry zeros)
      {
        uint32_t lw, dw;
        if constexpr (!WORDS_LDS) {
          lw = lw_next;
          dw = dw_next;
        } else {
          lw = nl[32 * jt + perm32(kl)];
          dw = nd[32 * jt + perm32(kl)];
        }
        s_off.set_raw(g ? 0u : lw);
        d_off.v[0] = g ? 0u : dw;
      }
      frag qn[DS], don[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        if constexpr (!FLAGGED) qn[s] = ofq.natural(qt, s);
        don[s] = ofq.natural(dot, s);
      }
      // Q^T, dO^T (A operands of dk, dv): transposing reads are the slowest LDS reads and the
      // four waves share one LDS pipe, so they are read once per query tile where registers
      // allow and again for every key tile where they do not
      constexpr bool QD_ONCE = D <= 32;
      frag qtr[DM][PS], dotr[DM][PS];
      auto load_qd_tr = [&] {
#pragma unroll
        for (int mt = 0; mt < DM; ++mt)
#pragma unroll
          for (int s2 = 0; s2 < PS; ++s2) {
            qtr[mt][s2] = ofq.transposed(qt, s2, mt);
            dotr[mt][s2] = ofq.transposed(dot, s2, mt);
          }
      };

      // ---- the state that moves from step to step --------------------------------------
      f32x16 s_cur, p_cur;   // scores and dP of the tile whose P, dS the step computes
      f32x16 s_nxt, p_nxt;   // ... of the tile after it, accumulating
      float p[16], ds[16];
      frag kn[DS];           // K rows of the next tile as B operand
      frag pf[PS], dsf[PS];  // P and dS of the last finished tile as B operands
      frag dst_prev[PS], ktr_prev[DM][PS];
      frag vn[DS];           // V operands of the next tile when they live in LDS
      auto load_kn = [&](int t) {
        if constexpr (!FLAGGED) {
          const unsigned char* ktile = lds_k + NWV * t * 32 * ROWB;
#pragma unroll
          for (int s = 0; s < DS; ++s) kn[s] = ofk.natural(ktile, s);
        }
      };
      load_kn(0);

      // Step t (t = -1 .. KT): the vector work of tile t (P, dS, their conversions) between
      // the MFMAs of its neighbours: dv, dk and dq of tile t-1, scores and dP of tile t+1,
      // in the order of RowSched.  Step -1 only starts tile 0, step KT only finishes tile KT-1.
      auto step = [&](auto tc) __attribute__((always_inline)) {
        constexpr int t = decltype(tc)::value - 1;
        constexpr bool has_prev = t >= 1, has_next = t + 1 < KT, valu = t >= 0 && t < KT;
        constexpr int tn = has_next ? t + 1 : 0, tp = has_prev ? t - 1 : 0;
        using Sch = RowSchedOf<has_prev, has_next, FLAGGED, NSB, DS, NACC, NDQ>;
        constexpr int NM = Sch::value.n;
        constexpr int NU = valu ? 16 : 0;  // vector units of four instructions
        // Step KT-2 starts the query tile after next on its way to LDS, right after its last
        // read of bias words: loads return in issue order,
        // so the next wait for bias words is a wait for these loads too, and from there it is
        // the furthest away, at the start of the next query tile.
        constexpr bool refill = t == KT - 2;
        constexpr int refill_at = FLAGGED ? 0 : Sch::value.last_sb;
        SB();
        TRI_ROW_TICK(t + 1);  // (slot 0: from the loop head to step -1; slot k: step k-2)
        // (words from the global planes: those of the next query tile, fetched before the last
        // bias tile of this one so that no wait for them is a wait for everything in flight)
        if constexpr (!WORDS_LDS && t == KT - 1) fetch_words(jt + 1, lw_next, dw_next);
        if constexpr (valu && !refill) fetch_bias(jt, t + 2);
        frag kb = keys_op.plain();
        if constexpr (has_next && MASKED) kb = keys_op.masked(kw[tn]);
        SB();
        static_for<NM>([&](auto xc) __attribute__((always_inline)) {
          constexpr int x = decltype(xc)::value;
          constexpr int kind = Sch::value.kind[x], idx = Sch::value.idx[x];
          if constexpr (kind == R_SOFF) {
            s_nxt = E::mfma(s_off.get(), kb, zero16());
          } else if constexpr (kind == R_SB) {
            s_nxt = E::mfma(__builtin_bit_cast(frag, bias_ring[tn % 2][idx / NPART]), bsel[idx / NPART][idx % NPART], s_nxt);
          } else if constexpr (kind == R_SQK) {
            s_nxt = E::mfma(qn[idx], kn[idx], s_nxt);
          } else if constexpr (kind == R_DOFF) {
            p_nxt = E::mfma(__builtin_bit_cast(frag, d_off.v), kb, zero16());
          } else if constexpr (kind == R_DP) {
            if constexpr (tn < VR) p_nxt = E::mfma(don[idx], vf[tn][idx], p_nxt);
            else p_nxt = E::mfma(don[idx], vn[idx], p_nxt);
          } else if constexpr (kind == R_ACC) {
            constexpr int s2 = (idx / 2) / DM, mt = (idx / 2) % DM;
            if constexpr (idx % 2 == 0) E::mfma_acc(dotr[mt][s2], pf[s2], dvacc[tp][mt]);
            else E::mfma_acc(qtr[mt][s2], dsf[s2], dkacc[tp][mt]);
          } else {
            if constexpr (tp == 0 && idx / DM == 0) dqacc[idx % DM] = E::mfma(ktr_prev[idx % DM][idx / DM], dst_prev[idx / DM], zero16());
            else dqacc[idx % DM] = E::mfma(ktr_prev[idx % DM][idx / DM], dst_prev[idx / DM], dqacc[idx % DM]);
          }
          SB();
          // Q^T, dO^T of the query tile are first used by the step after next: their reads go
          // where the LDS pipe has nothing else to do
          if constexpr (QD_ONCE && t == -1 && x == 1) load_qd_tr();
          // dq of the query tile before this one: its parts come from LDS early in this step,
          // which has no vector work of its own, and are summed and stored piece by piece behind
          // the MFMAs that follow (before the first query tile the sum is of stale bytes and is
          // not stored).  No wait for a load that could follow within the time a store takes
          // allows fewer than two operations in flight, so none of them waits for this store
          // (a wait for loads issued after a store is a wait for the store as well).
          if constexpr (t == -1) {
            if constexpr (x == 0) load_partials((jt + 1) & 1, parts);
#pragma unroll
            for (int piece = 0; piece < kSumPieces; ++piece)
              if ((piece + 3 < NM ? piece + 3 : NM - 1) == x) sum_dq_piece(piece, jt - 1, parts, carry, dq_words);
            if constexpr (x == NM - 1) {
              store_dq(jt - 1, dq_base, dq_words);
              if (jt > 0) dq_base += 32 * a.sdq.j;
              if constexpr (MULTI) {
                if (!first_pass) fetch_carry(jt, carry);
              }
            }
          }
          if constexpr (has_prev && x == Sch::value.dq_reads_at) {
            // dS of tile t-1 comes back from LDS with the key index in-lane, with the K
            // rows of that tile transposed beside it
            const unsigned char* ktile = lds_k + NWV * tp * 32 * ROWB;
#pragma unroll
            for (int s2 = 0; s2 < PS; ++s2) {
              dst_prev[s2] = ofd.transposed(ds_tile, s2, 0);
#pragma unroll
              for (int mt = 0; mt < DM; ++mt) ktr_prev[mt][s2] = ofk.transposed(ktile, s2, mt);
            }
          }
          if constexpr (refill && x == refill_at) {
            // (the last query tiles fetch the last one again, into a stage nobody reads any more)
            issue_stage(min(jt + 2, NJ - 1), buf_fill);
            fetch_bias(jt, t + 2);
          }
          if constexpr (has_next && x == Sch::value.last_sqk && t + 2 < KT) load_kn(t + 2);
          if constexpr (has_next && tn >= VR && x == Sch::value.v_reads_at) {
#pragma unroll
            for (int s = 0; s < DS; ++s) vn[s] = v_lds[((tn - VR) * DS + s) * 64];
          }
#pragma unroll
          for (int u = x * NU / NM; u < (x + 1) * NU / NM; ++u) {
            if (u < 8) {
#pragma unroll
              for (int e = 0; e < 2; ++e) p[2 * u + e] = fast_exp2(s_cur[2 * u + e] * c);
            } else if (u < 12) {
#pragma unroll
              for (int e = 0; e < 4; ++e) ds[4 * (u - 8) + e] = p[4 * (u - 8) + e] * p_cur[4 * (u - 8) + e];
            } else if (u < 14) {
              pf[u - 12] = E::pack(&p[KP * (u - 12)]);
            } else {
              dsf[u - 14] = E::pack(&ds[KP * (u - 14)]);
            }
          }
          SB();
        });
        if constexpr (valu) {
          // dS -> one of the wave's two LDS tiles [key][query]; Q^T, dO^T for the dv, dk
          // MFMAs of this tile, which the next step starts with
          *reinterpret_cast<frag*>(ds_tile + ds_w0) = dsf[0];
          *reinterpret_cast<frag*>(ds_tile + ds_w1) = dsf[1];
          if constexpr (!QD_ONCE) load_qd_tr();
          SB();
        }
        if constexpr (has_next) { s_cur = s_nxt; p_cur = p_nxt; }
      };
      static_for<KT + 2>(step);
      TRI_ROW_TICK(KT + 2);
      store_partials(jt & 1, dqacc);
      TRI_ROW_TICK(KT + 3);
      // The stage of the next query tile was requested a whole query tile ago; since then
      // the wave has issued the loads of the stage after it and (unless the row is fully
      // masked) of two bias tiles: everything older than those has landed.  A barrier
      // without a fence: a fence would wait for the loads in flight.  It is the only one of
      // the query tile: the partials written before it are read after it, and the buffer they
      // are in is written again two query tiles on, behind the next barrier.
      ring_sync<G2W + (FLAGGED ? 0 : 4) + (WORDS_LDS ? 0 : 2)>();
      TRI_ROW_TICK(KT + 4);
      buf = buf == 2 ? 0 : buf + 1;
    }
    {
      DqParts parts;
      DqOut dq_words;
      load_partials((NJ - 1) & 1, parts);
#pragma unroll
      for (int piece = 0; piece < kSumPieces; ++piece) sum_dq_piece(piece, NJ - 1, parts, carry, dq_words);
      store_dq(NJ - 1, dq_base, dq_words);
    }
#ifdef TRI_ROW_TIMING
    const uint64_t t_clk1 = __builtin_amdgcn_s_memtime(), t_loop1 = __builtin_amdgcn_s_memrealtime();
#endif

    // ---- dk, dv of this wave's keys -------------------------------------------------------
    // (the accumulators were last written by MFMAs inside asm statements, which the compiler
    // does not know to be MFMAs: each is read only after that MFMA has had time to retire)
    T* dkrow = reinterpret_cast<T*>(a.dk) + b * a.sdk.b + h * a.sdk.h + i * a.sdk.i;
    T* dvrow = reinterpret_cast<T*>(a.dv) + b * a.sdv.b + h * a.sdv.h + i * a.sdv.i;
  #pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int key = 32 * (KT0 + NWV * t + wave) + kl;
  #pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
#ifndef TRI_MFMA_ACC_BUILTIN
        asm volatile("s_nop 15" : "+a"(dkacc[t][mt]));
        asm volatile("s_nop 15" : "+a"(dvacc[t][mt]));
#endif
      }
      store_rows_wide<T, D, DM>(dkrow + (int64_t)key * a.sdk.j, dkacc[t], a.scale, g, key < N);
      store_rows_wide<T, D, DM>(dvrow + (int64_t)key * a.sdv.j, dvacc[t], 1.0f, g, key < N);
    }
#ifdef TRI_ROW_TIMING
    // one record of 32 words per workgroup (wave 0), at the start of what db points to
    if (wave == 0 && lane == 0) {
      uint64_t* rec = reinterpret_cast<uint64_t*>(a.db) + (int64_t)L * 32;
      const uint64_t t_end = __builtin_amdgcn_s_memrealtime();
      const uint64_t marks[8] = {t_entry, t_p1, t_p2, t_p3, t_p4, t_loop0, t_loop1, t_end};  // 100 MHz
      for (int x = 0; x < 8; ++x) rec[x] = marks[x];
      rec[8] = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (31 << 11));   // HW_ID
      rec[9] = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (31 << 11));  // XCC_ID
      rec[10] = t_clk1 - t_clk0;                                        // shader clocks of the loop
      for (int x = 0; x < KT + 5; ++x) rec[11 + x] = tacc[x];
    }
#endif
  };
  bool plain = true;
#pragma unroll
  for (int t = 0; t < KT; ++t) plain = plain && kw[t] == 0xffffffffu;
  if (flagged) query_tiles(std::true_type{}, std::true_type{});
  else if (plain) query_tiles(std::false_type{}, std::false_type{});
  else query_tiles(std::true_type{}, std::false_type{});

}

}  // namespace tri
