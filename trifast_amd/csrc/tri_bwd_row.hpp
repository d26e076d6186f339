// Row-resident backward: dq, dk and dv of one pair row from ONE computation of the
// scores and of dP (the dq kernel and the dk/dv kernel each recompute both).
//
// Work unit: (batch*head, pair row i), one workgroup of four waves, one wave per
// SIMD with the whole register file.  The keys of the row are dealt to the waves
// in tiles of 32 (wave w owns key tiles w, w+4, ...; at most KT of them): their
// dk, dv accumulators stay in registers for the whole row, their V rows too (B
// operands), and the K row of the pair row sits in LDS for the whole workgroup
// (read as B operand of the scores and, transposed, as A operand of dq).  The
// queries of the row are streamed through LDS in tiles of 32 (Q, dO rows, direct
// global->LDS loads, double-buffered).  Per (query tile, key tile), with the
// scores un-transposed (a lane owns one key and 16 queries):
//   S  = Q K^T + sqrt(d) (bias - lse)      bias tile -> fp32 once, as accumulator init
//   P  = exp2(c S)
//   dP = dO V^T - delta                    -delta as accumulator init
//   dS = P * dP
//   dv^T += dO^T P,  dk^T += Q^T dS        P, dS are B operands as they are
//   dq^T += K^T dS^T                       dS goes through a 2 KiB LDS tile of the wave
//                                          and comes back transposed (ds_read_tr)
// The per-query terms (-lse sqrt(d), -delta) are the same for every key tile of a
// query tile: the 16 values a lane needs are loaded once per query tile and enter
// as accumulator inits, so no rank-1 MFMA and no add is spent on them.  dq of a
// query tile is the sum of the four waves' partial tiles: they meet in LDS once
// per query tile and are added in wave order (deterministic, no atomics).
//
// The prologue also computes delta = rowsum(o * do) of the row and leaves it, with
// the row's log-sum-exp, in the per-query planes the db kernel reads.
//
// Rows up to 128*KT keys fit (1024 keys at head dim 32); longer rows use the dq and
// dk/dv kernels.  Replaces _bwd_q and _bwd_kv of reference
// src/trifast/triton.py:274-383 and :143-263 in one pass.
#pragma once
#include <type_traits>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

constexpr int kRowWaves = 4;

// LDS bytes of the kernel below
constexpr int bwd_row_base_lds_bytes(int D, int es, int KT) {
  const int rowb = D * es, dm = (D + 31) / 32, keys = kRowWaves * KT * 32;
  const int nred = dm == 1 ? 2 : 1;
  return keys * rowb + 2 * (2 * 32 * rowb) + kRowWaves * 2 * 2048 + nred * kRowWaves * dm * 4096 + 2 * keys * 4;
}
// query tiles per half of the dq staging buffer: what is left of the 160 KiB, at most 8
constexpr int bwd_row_dq_half(int D, int es, int KT) {
  const int left = (160 * 1024 - bwd_row_base_lds_bytes(D, es, KT)) / (2 * 32 * D * es);
  return left > 8 ? 8 : left;
}
constexpr int bwd_row_lds_bytes(int D, int es, int KT) {
  return bwd_row_base_lds_bytes(D, es, KT) + 2 * bwd_row_dq_half(D, es, KT) * 32 * D * es;
}

template <typename T, int D, int KT>
__global__ __launch_bounds__(kRowWaves * 64, 1) void tri_bwd_row_kernel(const BwdArgs a) {
  static_assert(sizeof(T) == 2, "16-bit inputs only (the transposing LDS reads)");
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  using DsTile = LdsTile<T, 32>;
  constexpr int NWV = kRowWaves;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 2;
  constexpr int ROWB = Tile::ROWB;
  constexpr int KEYS = NWV * KT * 32;         // keys (and queries) the workgroup can hold
  constexpr int NRED = DM == 1 ? 2 : 1;       // dq partial buffers (two: one barrier per query tile)
  constexpr int STAGE = 2 * 32 * ROWB;        // Q tile | dO tile
  constexpr int OFF_K = 0;
  constexpr int OFF_ST = KEYS * ROWB;
  constexpr int OFF_DS = OFF_ST + 2 * STAGE;
  constexpr int OFF_RED = OFF_DS + NWV * 2 * 2048;
  constexpr int OFF_NL = OFF_RED + NRED * NWV * DM * 4096;
  constexpr int OFF_ND = OFF_NL + KEYS * 4;
  // finished dq rows wait here in two halves of DQH query tiles each and leave in bursts of
  // whole rows: stores inside the tile loop would make every wait for a load a wait for
  // all memory traffic in flight (loads and stores retire out of order with each other)
  constexpr int DQH = bwd_row_dq_half(D, (int)sizeof(T), KT);
  static_assert(DQH >= 1, "no room for the dq staging buffer");
  constexpr int OFF_DQ = OFF_ND + KEYS * 4;
  static_assert(OFF_DQ + 2 * DQH * 32 * ROWB == bwd_row_lds_bytes(D, (int)sizeof(T), KT), "the launcher sizes LDS with bwd_row_lds_bytes");
  static_assert((KT - 1) * NWV * 32 * ROWB + 32 * ROWB <= 65536, "key tile offsets are LDS immediates");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kl = lane & 31, g = lane >> 5;
  const int N = a.N;
  const int NJ = a.nwords;  // 32-tiles of the row (queries and keys)

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
  const T* pack_bh = reinterpret_cast<const T*>(a.packk) + (int64_t)bh * a.NP * a.NP * 1024;

  unsigned char* const lds_k = tri_smem + OFF_K;
  float* const nl = reinterpret_cast<float*>(tri_smem + OFF_NL);
  float* const nd = reinterpret_cast<float*>(tri_smem + OFF_ND);

  // ---- prologue -----------------------------------------------------------------
  // K row -> LDS (rows past the end repeat the last key; their keep bits are clear)
  Tile::template fill<KEYS, NWV>(lds_k, [&](int r) { return krow + (int64_t)min(r, N - 1) * a.sk.j; }, wave, lane);
  // query tiles 0 (and 1) -> the two stage buffers
  // (per-lane source pointers for query tile 0, computed once; a tile inside the row adds
  // one uniform offset, the ragged last one clamps the query index)
  auto issue_stage = [&](int jt, int buf) {
    unsigned char* st = tri_smem + OFF_ST + buf * STAGE;
    if (32 * jt + 32 <= N) {
      // (the source addresses are rebuilt from the lane id every time: kept in registers
      // from one query tile to the next they would be spilled, and a reload from scratch
      // waits for every load in flight)
      int lane_now = lane;
      asm volatile("" : "+v"(lane_now));  // (opaque: nothing derived from it is hoisted out of the loop)
      Tile::template fill<32, NWV>(st, [&](int r) { return qrow + (int64_t)(32 * jt + r) * a.sq.j; }, wave, lane_now);
      Tile::template fill<32, NWV>(st + 32 * ROWB, [&](int r) { return dorow + (int64_t)(32 * jt + r) * a.sdo.j; }, wave, lane_now);
    } else {
      asm volatile("" ::);  // keeps this rare path a real branch
      Tile::template fill<32, NWV>(st, [&](int r) { return qrow + (int64_t)min(32 * jt + r, N - 1) * a.sq.j; }, wave, lane);
      Tile::template fill<32, NWV>(st + 32 * ROWB, [&](int r) { return dorow + (int64_t)min(32 * jt + r, N - 1) * a.sdo.j; }, wave, lane);
    }
  };
  issue_stage(0, 0);

  // a fully masked row drops q.k and the bias from its scores (all logits equal)
  const bool flagged = __builtin_amdgcn_readfirstlane(a.rowflag[(int64_t)b * N + i]) != 0;
  // keep words of this wave's key tiles (bit k set = key k of the tile is attended)
  uint32_t kw[KT];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int kt = NWV * t + wave;
    kw[t] = __builtin_amdgcn_readfirstlane(kt < NJ ? a.keep[((int64_t)b * N + i) * a.nwords + kt] : 0u);
  }
  const uint32_t lanebit = 1u << kl;

  // V rows of this lane's keys as B operands
  frag vf[KT][DS];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int key = min(32 * (NWV * t + wave) + kl, N - 1);
#pragma unroll
    for (int s = 0; s < DS; ++s) vf[t][s] = *reinterpret_cast<const frag*>(vrow + (int64_t)key * a.sv.j + 2 * KP * s + KP * g);
  }

  // per-query terms of the row: -delta and -lse*sqrt(d) (ln n for lse in a fully masked
  // row), kept in LDS for this kernel and written as MFMA operand words for the db kernel
  {
    const T* orow = reinterpret_cast<const T*>(a.o) + ((int64_t)bh * N + i) * N * D;
    const float* lserow = a.lse + ((int64_t)bh * N + i) * N;
    uint32_t* dplane = a.delta + ((int64_t)bh * N + i) * N;
    uint32_t* lplane = a.lse2 + ((int64_t)bh * N + i) * N;
    const float flat = -__builtin_amdgcn_logf((float)N) * (kLn2 * a.sqrt_d);
    for (int j = tid; j < KEYS; j += NWV * 64) {
      float nlv = kNeg, ndv = 0.f;  // queries past the end: P = dS = 0
      if (j < N) {
        float dsum = 0.f;
#pragma unroll
        for (int s = 0; s < D / 8; ++s) {
          const typename E::vec ov = *reinterpret_cast<const typename E::vec*>(orow + (int64_t)j * D + 8 * s);
          const typename E::vec dv = *reinterpret_cast<const typename E::vec*>(dorow + (int64_t)j * a.sdo.j + 8 * s);
#pragma unroll
          for (int e = 0; e < 8; ++e) dsum += (float)ov[e] * (float)dv[e];
        }
        ndv = -dsum;
        nlv = flagged ? flat : -lserow[j] * a.sqrt_d;
        dplane[j] = split_word<T>(ndv);
        lplane[j] = split_word<T>(nlv);
      }
      nl[j] = nlv;
      nd[j] = ndv;
    }
  }

  // lane-constant LDS offsets.  Q, dO tiles: natural A operands (tile row m stands for
  // query perm32(m)) and transposed A operands; K tiles: natural B operand of this lane's
  // key and transposed A operand; the wave's dS tile: write offsets and transposed reads.
  OperandOffsets<T, D> ofq, ofk;
  ofq.init(perm32(kl), lane);
  ofk.init(kl, lane);
  ofk.shift(wave * 32 * ROWB);  // key tile t of this wave starts (4 t + wave) * 32 rows into K
  OperandOffsets<T, 32> ofd;
  ofd.init(0, lane);
  unsigned char* const ds_tile = tri_smem + OFF_DS + wave * 2 * 2048;  // two tiles, used in turn
  const int ds_w0 = DsTile::off(kl, 16 * g), ds_w1 = DsTile::off(kl, 32 + 16 * g);


  // packed bias tiles of this lane: tile (jt, kt) is 2 x 16 bytes per lane
  typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
  const T* bias_lane = pack_bh + lane * 8;
  auto bias_load = [&](int jt, int t, u32x4v* dst) {
    const int kt = min(NWV * t + wave, a.NP - 1);
    const T* p = bias_lane + ((int64_t)min(jt, a.NP - 1) * a.NP + kt) * 1024;
    dst[0] = *reinterpret_cast<const u32x4v*>(p);
    dst[1] = *reinterpret_cast<const u32x4v*>(p + 512);
  };
  const float c = a.c;
  const float a_sqrt_d = a.sqrt_d;

  // dq partial tiles of the four waves: [buffer][wave][mt][quarter][lane] x 16 bytes
  auto red_slot = [&](int buf, int w, int mt, int q) -> f32x4* {
    return reinterpret_cast<f32x4*>(tri_smem + OFF_RED + (((buf * NWV + w) * DM + mt) * 4 + q) * 1024) + lane;
  };
  // sum the partials of query tile jt in wave order; this wave owns quarter `wave` of
  // every lane's values: head-dim elements 32 mt + 8 wave + 4 g + 0..3 of query 32 jt + kl
  // (the finished elements go to the dq staging buffer: row-major rows of D elements, query
  // tile jt in slot jt % (2 DQH))
  T* dqrow = reinterpret_cast<T*>(a.dq) + b * a.sdq.b + h * a.sdq.h + i * a.sdq.i;
  auto reduce_dq = [&](int jt, int buf) {
    T* slot = reinterpret_cast<T*>(tri_smem + OFF_DQ) + ((jt % (2 * DQH)) * 32 + kl) * D;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      const int d0 = 32 * mt + 8 * wave + 4 * g;
      f32x4 acc = *red_slot(buf, 0, mt, wave);
#pragma unroll
      for (int w = 1; w < NWV; ++w) acc += *red_slot(buf, w, mt, wave);
      if (d0 < D) {
        typename E::vec4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (T)(acc[e] * a.scale);
        *reinterpret_cast<typename E::vec4*>(slot + d0) = ov;
      }
    }
  };
  // write query tiles [jt0, jt1) of the staging buffer to dq: whole rows, 16 bytes per lane
  auto flush_dq = [&](int jt0, int jt1) {
    constexpr int CPR = Tile::CPR;
    const int chunks = (jt1 - jt0) * 32 * CPR;
    for (int cidx_ = tid; cidx_ < chunks; cidx_ += NWV * 64) {
      const int row = cidx_ / CPR, col = cidx_ % CPR;
      const int j = 32 * jt0 + row;
      if (j >= N) break;
      const T* src = reinterpret_cast<const T*>(tri_smem + OFF_DQ) + ((j % (2 * DQH * 32)) * D + col * Tile::VEC);
      *reinterpret_cast<typename E::vec*>(dqrow + (int64_t)j * a.sdq.j + col * Tile::VEC) = *reinterpret_cast<const typename E::vec*>(src);
    }
  };

  wait_dma();
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
    static_assert(KT % 2 == 0, "the two-slot bias ring assumes an even number of key tiles per wave");
    // The wave is alone on its SIMD, so nothing but its own instruction order hides a
    // latency: the code below is laid out as the schedule it should run in, and scheduling
    // barriers between the pieces keep the compiler from re-ordering it.
    auto SB = [] { __builtin_amdgcn_sched_barrier(0); };
    constexpr int NACC = 2 * PS * DM;  // dv, dk MFMAs of a tile
    constexpr int NDQ = PS * DM;       // dq MFMAs of a tile
    // packed bias of key tile t (t >= KT: tile t - KT of the next query tile) -> ring slot t % 2,
    // fetched two steps before its use (global memory, through L2)
    u32x4v bias_ring[2][2] = {};
    auto fetch_bias = [&](int jt, int t) {
#ifndef TRI_ABL_NOBIAS
      bias_load(jt + t / KT, t % KT, bias_ring[t % 2]);
#endif
    };
    fetch_bias(0, 0);
    fetch_bias(0, 1);
#ifdef TRI_ROW_PROF
    uint64_t prof[8] = {};
    const uint64_t tstart = __builtin_amdgcn_s_memtime();
    uint64_t tlast = tstart;
#define TRI_TS(k) { SB(); const uint64_t now = __builtin_amdgcn_s_memtime(); prof[k] += now - tlast; tlast = now; SB(); }
#else
#define TRI_TS(k)
#endif
    for (int jt = 0; jt < NJ; ++jt) {
      const int buf = jt & 1;
      if (jt + 1 < NJ) issue_stage(jt + 1, buf ^ 1);
      // the half of the staging buffer whose last query tile was reduced one iteration
      // ago (and published by the barrier since) leaves now
      if (jt >= DQH + 1 && (jt - 1) % DQH == 0) {
        asm volatile("" ::);  // a real branch: taken once in DQH iterations
        flush_dq(jt - 1 - DQH, jt - 1);
      }
      if (jt > 0) {
        if constexpr (NRED == 2) reduce_dq(jt - 1, (jt - 1) & 1);
      }
      const unsigned char* qt = tri_smem + OFF_ST + buf * STAGE;
      const unsigned char* dot = qt + 32 * ROWB;

      // the 16 queries of this lane's values: 8 g + 0..7 and 16 + 8 g + 0..7 of the tile
      f32x16 nlse, ndelta;
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int q4 = 0; q4 < 2; ++q4) {
          const f32x4 x = *reinterpret_cast<const f32x4*>(nl + 32 * jt + 16 * r + 8 * g + 4 * q4);
          const f32x4 y = *reinterpret_cast<const f32x4*>(nd + 32 * jt + 16 * r + 8 * g + 4 * q4);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            nlse[8 * r + 4 * q4 + e] = x[e];
            ndelta[8 * r + 4 * q4 + e] = y[e];
          }
        }
      frag qn[DS], don[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        if constexpr (!FLAGGED) qn[s] = ofq.natural(qt, s);
        don[s] = ofq.natural(dot, s);
      }
      // Q^T, dO^T (A operands of dk, dv) are read again for every key tile, right before
      // the step that uses them: held for the whole query tile they would be 8 DM registers
      // too many at the point where most values are live
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
      f32x16 dqacc[DM];
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) dqacc[mt] = zero16();
      TRI_TS(0)

      // ---- the pieces of one key tile's work -------------------------------------------
      // quarter a of the score accumulator init of a tile: sqrt(d) * bias - lse * sqrt(d)
      // (a large negative bias for masked keys and keys past the end); 8 vector instructions
      auto init_quarter = [&](int a, int t, f32x16& sc) {
        if constexpr (FLAGGED) {
#pragma unroll
          for (int e = 0; e < 4; ++e) sc[4 * a + e] = nlse[4 * a + e];  // all logits of the row are equal
        } else {
          uint32_t w[2] = {bias_ring[t % 2][a / 2][2 * (a % 2)], bias_ring[t % 2][a / 2][2 * (a % 2) + 1]};
          if constexpr (MASKED) {
            const bool kept = (kw[t] & lanebit) != 0;
            constexpr uint32_t kMaskPair = (std::is_same<T, __bf16>::value ? 0xf149u : 0xf0e2u) * 0x10001u;  // two bf16 of -1e30 / fp16 of -10000
            w[0] = kept ? w[0] : kMaskPair;
            w[1] = kept ? w[1] : kMaskPair;
          }
          typedef T pair_t __attribute__((ext_vector_type(2)));
#pragma unroll
          for (int x = 0; x < 2; ++x) {
            const pair_t pr = __builtin_bit_cast(pair_t, w[x]);
            sc[4 * a + 2 * x] = __builtin_fmaf((float)pr[0], a_sqrt_d, nlse[4 * a + 2 * x]);
            sc[4 * a + 2 * x + 1] = __builtin_fmaf((float)pr[1], a_sqrt_d, nlse[4 * a + 2 * x + 1]);
          }
        }
      };
      float p[16], ds[16];
      // quarter bq of P = exp2(c * scores); 8 vector instructions
      auto p_quarter = [&](int bq, int t, const f32x16& sc) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
#ifdef TRI_ABL_NOEXP
          p[4 * bq + e] = sc[4 * bq + e] * c;
#else
          p[4 * bq + e] = fast_exp2(sc[4 * bq + e] * c);
#endif
        }
        if constexpr (FLAGGED) {
          // keys past the end of the row stay out of a fully masked row too
          const bool kept = (kw[t] & lanebit) != 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) p[4 * bq + e] = kept ? p[4 * bq + e] : 0.f;
        }
      };
      // half cq of dS = P * (dP - delta); 8 vector instructions
      auto ds_half = [&](int cq, const f32x16& dp) {
#pragma unroll
        for (int e = 0; e < 8; ++e) ds[8 * cq + e] = p[8 * cq + e] * dp[8 * cq + e];
      };
      frag kn[DS];       // K rows of the next tile as B operand
      frag pf[PS], dsf[PS];  // P and dS of the last finished tile as B operands
      auto load_kn = [&](int t) {
        const unsigned char* ktile = lds_k + NWV * t * 32 * ROWB;
#pragma unroll
        for (int s = 0; s < DS; ++s) kn[s] = ofk.natural(ktile, s);
      };
      // dv, dk MFMA number x of tile t (x = 2 (s2 DM + mt) + {0: dv, 1: dk})
      auto acc_mfma = [&](int t, int x) {
        const int s2 = (x / 2) / DM, mt = (x / 2) % DM;
#ifndef TRI_ABL_NOACC
        if (x % 2 == 0) E::mfma_acc(dotr[mt][s2], pf[s2], dvacc[t][mt]);
        else E::mfma_acc(qtr[mt][s2], dsf[s2], dkacc[t][mt]);
#endif
      };

      // ---- tile 0: scores and dP with nothing to run beside them -------------------------
      f32x16 s_cur, p_cur;
      load_kn(0);
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) init_quarter(a4, 0, s_cur);
      p_cur = ndelta;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        if constexpr (!FLAGGED) s_cur = E::mfma(qn[s], kn[s], s_cur);
        p_cur = E::mfma(don[s], vf[0][s], p_cur);
      }
      load_kn(1);
      TRI_TS(2)

      // ---- step t: P, dS of tile t (vector ALU) beside the MFMAs of its neighbours: dv, dk
      // of tile t-1, scores and dP of tile t+1, dq of tile t-1 ------------------------------
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        const bool has_next = t + 1 < KT;
        f32x16 s_nxt, p_nxt;
        frag dst_prev[PS], ktr_prev[DM][PS];
        SB();
        fetch_bias(jt, t + 2);
        SB();
        // score init of tile t+1 | dv, dk of tile t-1
#pragma unroll
        for (int a4 = 0; a4 < 4; ++a4) {
          if (t >= 1) {
#pragma unroll
            for (int x = a4 * NACC / 4; x < (a4 + 1) * NACC / 4; ++x) acc_mfma(t - 1, x);
            if (a4 == 2) {
              // dS of tile t-1 comes back from LDS with the key index in-lane, with the K
              // rows of that tile transposed beside it (for dq, two slots further down)
              const unsigned char* ktile = lds_k + NWV * (t - 1) * 32 * ROWB;
              const unsigned char* src = ds_tile + ((t - 1) & 1) * 2048;
#pragma unroll
              for (int s2 = 0; s2 < PS; ++s2) {
#ifdef TRI_ABL_NODS
                dst_prev[s2] = qn[s2 % DS];
#else
                dst_prev[s2] = ofd.transposed(src, s2, 0);
#endif
#pragma unroll
                for (int mt = 0; mt < DM; ++mt) ktr_prev[mt][s2] = ofk.transposed(ktile, s2, mt);
              }
            }
          }
          SB();
          if (has_next) init_quarter(a4, t + 1, s_nxt);
          SB();
        }
        // P of tile t | scores of tile t+1, then dq of tile t-1
#pragma unroll
        for (int bq = 0; bq < 4; ++bq) {
          if (bq < 2) {
            if constexpr (!FLAGGED) {
              if (has_next) {
#pragma unroll
                for (int s = bq * DS / 2; s < (bq + 1) * DS / 2; ++s) s_nxt = E::mfma(qn[s], kn[s], s_nxt);
              }
            }
          } else {
#ifndef TRI_ABL_NODQ
            if (t >= 1) {
#pragma unroll
              for (int x = (bq - 2) * NDQ / 2; x < (bq - 1) * NDQ / 2; ++x)
                dqacc[x % DM] = E::mfma(ktr_prev[x % DM][x / DM], dst_prev[x / DM], dqacc[x % DM]);
            }
#endif
          }
          SB();
          p_quarter(bq, t, s_cur);
          SB();
        }
        if (t + 2 < KT) load_kn(t + 2);
        // dS of tile t | dP of tile t+1
#pragma unroll
        for (int cq = 0; cq < 2; ++cq) {
          if (has_next) {
#pragma unroll
            for (int s = cq * DS / 2; s < (cq + 1) * DS / 2; ++s) p_nxt = E::mfma(don[s], vf[(t + 1) % KT][s], s == 0 ? ndelta : p_nxt);
          }
          SB();
          ds_half(cq, p_cur);
          SB();
        }
        // P, dS -> B operands; dS -> one of the wave's two LDS tiles [key][query]
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) pf[s2] = E::pack(&p[KP * s2]);
        SB();
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) dsf[s2] = E::pack(&ds[KP * s2]);
        {
          unsigned char* dst = ds_tile + (t & 1) * 2048;
          *reinterpret_cast<frag*>(dst + ds_w0) = dsf[0];
          *reinterpret_cast<frag*>(dst + ds_w1) = dsf[1];
        }
        load_qd_tr();  // for the dv, dk MFMAs of this tile, at the start of the next step
        SB();
        if (has_next) { s_cur = s_nxt; p_cur = p_nxt; }
      }
      TRI_TS(3)
      // ---- the last tile's dv, dk and dq ---------------------------------------------------
      {
        const unsigned char* ktile = lds_k + NWV * (KT - 1) * 32 * ROWB;
        const unsigned char* src = ds_tile + ((KT - 1) & 1) * 2048;
        frag dst_prev[PS], ktr_prev[DM][PS];
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          dst_prev[s2] = ofd.transposed(src, s2, 0);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) ktr_prev[mt][s2] = ofk.transposed(ktile, s2, mt);
        }
#pragma unroll
        for (int x = 0; x < NACC; ++x) acc_mfma(KT - 1, x);
#ifndef TRI_ABL_NODQ
#pragma unroll
        for (int x = 0; x < NDQ; ++x) dqacc[x % DM] = E::mfma(ktr_prev[x % DM][x / DM], dst_prev[x / DM], dqacc[x % DM]);
#endif
      }
      TRI_TS(4)

      // this wave's partial dq tile -> LDS
      const int rbuf = NRED == 2 ? buf : 0;
#pragma unroll
      for (int mt = 0; mt < DM; ++mt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          f32x4 x;
#pragma unroll
          for (int e = 0; e < 4; ++e) x[e] = dqacc[mt][4 * q + e];
          *red_slot(rbuf, wave, mt, q) = x;
        }
      TRI_TS(5)
      wait_dma();
      __syncthreads();
      TRI_TS(6)
      if constexpr (NRED == 1) {
        reduce_dq(jt, 0);
        __syncthreads();
      }
    }
    if constexpr (NRED == 2) reduce_dq(NJ - 1, (NJ - 1) & 1);
    // the query tiles still in the staging buffer: everything from the last flushed half on
    __syncthreads();
    flush_dq(NJ >= 2 ? (NJ - 2) / DQH * DQH : 0, NJ);
#ifdef TRI_ROW_PROF
    // phase cycle totals of wave 0 of the first workgroup -> the front of the db partial buffer
    if (blockIdx.x == 0 && wave == 0 && a.dbpart) {
      prof[7] = __builtin_amdgcn_s_memtime() - tstart;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk)
        if (lane == kk) reinterpret_cast<uint64_t*>(a.dbpart)[kk] = prof[kk];
    }
#endif

    // ---- dk, dv of this wave's keys -------------------------------------------------------
    // (the accumulators were last written by MFMAs inside asm statements, which the compiler
    // does not know to be MFMAs: each is read only after that MFMA has had time to retire)
    T* dkrow = reinterpret_cast<T*>(a.dk) + b * a.sdk.b + h * a.sdk.h + i * a.sdk.i;
    T* dvrow = reinterpret_cast<T*>(a.dv) + b * a.sdv.b + h * a.sdv.h + i * a.sdv.i;
  #pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int key = 32 * (NWV * t + wave) + kl;
  #pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        asm volatile("s_nop 15" : "+a"(dkacc[t][mt]));
        asm volatile("s_nop 15" : "+a"(dvacc[t][mt]));
      }
      if (key >= N) continue;
      store_rows<T, D, DM>(dkrow + (int64_t)key * a.sdk.j, dkacc[t], a.scale, g);
      store_rows<T, D, DM>(dvrow + (int64_t)key * a.sdv.j, dvacc[t], 1.0f, g);
    }
  };
  bool plain = true;
#pragma unroll
  for (int t = 0; t < KT; ++t) plain = plain && kw[t] == 0xffffffffu;
  if (flagged) query_tiles(std::true_type{}, std::true_type{});
  else if (plain) query_tiles(std::false_type{}, std::false_type{});
  else query_tiles(std::true_type{}, std::false_type{});

}

}  // namespace tri
