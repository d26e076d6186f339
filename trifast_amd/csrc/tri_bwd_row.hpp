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
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

constexpr int kRowWaves = 4;

// LDS bytes of the kernel below
constexpr int bwd_row_lds_bytes(int D, int es, int KT) {
  const int rowb = D * es, dm = (D + 31) / 32, keys = kRowWaves * KT * 32;
  const int nred = dm == 1 ? 2 : 1;
  return keys * rowb + 2 * (2 * 32 * rowb) + kRowWaves * 2048 + nred * kRowWaves * dm * 4096 + 2 * keys * 4;
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
  constexpr int OFF_RED = OFF_DS + NWV * 2048;
  constexpr int OFF_NL = OFF_RED + NRED * NWV * DM * 4096;
  constexpr int OFF_ND = OFF_NL + KEYS * 4;
  static_assert(OFF_ND + KEYS * 4 == bwd_row_lds_bytes(D, (int)sizeof(T), KT), "the launcher sizes LDS with bwd_row_lds_bytes");
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
  auto issue_stage = [&](int jt, int buf) {
    unsigned char* st = tri_smem + OFF_ST + buf * STAGE;
    Tile::template fill<32, NWV>(st, [&](int r) { return qrow + (int64_t)min(32 * jt + r, N - 1) * a.sq.j; }, wave, lane);
    Tile::template fill<32, NWV>(st + 32 * ROWB, [&](int r) { return dorow + (int64_t)min(32 * jt + r, N - 1) * a.sdo.j; }, wave, lane);
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
  unsigned char* const ds_tile = tri_smem + OFF_DS + wave * 2048;
  const int ds_w0 = DsTile::off(kl, 16 * g), ds_w1 = DsTile::off(kl, 32 + 16 * g);

  f32x16 dkacc[KT][DM], dvacc[KT][DM];
#pragma unroll
  for (int t = 0; t < KT; ++t)
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      E::mfma_acc_zero(dkacc[t][mt]);
      E::mfma_acc_zero(dvacc[t][mt]);
    }

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
  const float sqrt_d = flagged ? 0.f : a.sqrt_d;

  // dq partial tiles of the four waves: [buffer][wave][mt][quarter][lane] x 16 bytes
  auto red_slot = [&](int buf, int w, int mt, int q) -> f32x4* {
    return reinterpret_cast<f32x4*>(tri_smem + OFF_RED + (((buf * NWV + w) * DM + mt) * 4 + q) * 1024) + lane;
  };
  // sum the partials of query tile jt in wave order; this wave owns quarter `wave` of
  // every lane's values: head-dim elements 32 mt + 8 wave + 4 g + 0..3 of query 32 jt + kl
  T* dqrow = reinterpret_cast<T*>(a.dq) + b * a.sdq.b + h * a.sdq.h + i * a.sdq.i;
  auto reduce_dq = [&](int jt, int buf) {
    const int j = 32 * jt + kl;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      const int d0 = 32 * mt + 8 * wave + 4 * g;
      f32x4 acc = *red_slot(buf, 0, mt, wave);
#pragma unroll
      for (int w = 1; w < NWV; ++w) acc += *red_slot(buf, w, mt, wave);
      if (j < N && d0 < D) {
        typename E::vec4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (T)(acc[e] * a.scale);
        *reinterpret_cast<typename E::vec4*>(dqrow + (int64_t)j * a.sdq.j + d0) = ov;
      }
    }
  };

  u32x4v bias_next[2];
  bias_load(0, 0, bias_next);
  wait_dma();
  __syncthreads();

  // ---- query tiles ------------------------------------------------------------------
  for (int jt = 0; jt < NJ; ++jt) {
    const int buf = jt & 1;
    if (jt + 1 < NJ) issue_stage(jt + 1, buf ^ 1);
    if (jt > 0) {
      if constexpr (NRED == 2) {
        reduce_dq(jt - 1, (jt - 1) & 1);
      }
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
    frag qn[DS], don[DS], qs[DS], qtr[DM][PS], dotr[DM][PS];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      qn[s] = ofq.natural(qt, s);
      don[s] = ofq.natural(dot, s);
      qs[s] = flagged ? E::zero() : qn[s];
    }
#pragma unroll
    for (int mt = 0; mt < DM; ++mt)
#pragma unroll
      for (int s2 = 0; s2 < PS; ++s2) {
        qtr[mt][s2] = ofq.transposed(qt, s2, mt);
        dotr[mt][s2] = ofq.transposed(dot, s2, mt);
      }
    f32x16 dqacc[DM];
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) dqacc[mt] = zero16();

#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int kt = NWV * t + wave;
      // the next tile's bias is fetched while this one is worked on
      u32x4v braw[2] = {bias_next[0], bias_next[1]};
      if (t + 1 < KT) bias_load(jt, t + 1, bias_next);
      else bias_load(jt + 1, 0, bias_next);
      (void)kt;

      const unsigned char* ktile = lds_k + NWV * t * 32 * ROWB;
      // scores: sqrt(d) * bias - lse * sqrt(d) as accumulator init, then Q K^T
      f32x16 sc;
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const typename E::vec x = __builtin_bit_cast(typename E::vec, braw[r]);
#pragma unroll
        for (int e = 0; e < 8; ++e) sc[8 * r + e] = __builtin_fmaf((float)x[e], sqrt_d, nlse[8 * r + e]);
      }
      f32x16 dp = ndelta;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        sc = E::mfma(qs[s], ofk.natural(ktile, s), sc);
        dp = E::mfma(don[s], vf[t][s], dp);
      }
      float p[16], ds[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) p[v] = fast_exp2(sc[v] * c);
      if (kw[t] != 0xffffffffu) {
        // some keys of the tile are masked out (or lie past the end): their P is zero
        const bool kept = (kw[t] & lanebit) != 0;
#pragma unroll
        for (int v = 0; v < 16; ++v) p[v] = kept ? p[v] : 0.f;
      }
#pragma unroll
      for (int v = 0; v < 16; ++v) ds[v] = p[v] * dp[v];
      frag pf[PS], dsf[PS];
#pragma unroll
      for (int s2 = 0; s2 < PS; ++s2) {
        pf[s2] = E::pack(&p[KP * s2]);
        dsf[s2] = E::pack(&ds[KP * s2]);
      }
      // dS -> the wave's LDS tile [key][query], read back with the key index in-lane
      *reinterpret_cast<frag*>(ds_tile + ds_w0) = dsf[0];
      *reinterpret_cast<frag*>(ds_tile + ds_w1) = dsf[1];
#pragma unroll
      for (int s2 = 0; s2 < PS; ++s2)
#pragma unroll
        for (int mt = 0; mt < DM; ++mt) {
          E::mfma_acc(dotr[mt][s2], pf[s2], dvacc[t][mt]);
          E::mfma_acc(qtr[mt][s2], dsf[s2], dkacc[t][mt]);
        }
#pragma unroll
      for (int s2 = 0; s2 < PS; ++s2) {
        const frag dst = ofd.transposed(ds_tile, s2, 0);
#pragma unroll
        for (int mt = 0; mt < DM; ++mt) dqacc[mt] = E::mfma(ofk.transposed(ktile, s2, mt), dst, dqacc[mt]);
      }
    }

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
    wait_dma();
    __syncthreads();
    if constexpr (NRED == 1) {
      reduce_dq(jt, 0);
      __syncthreads();
    }
  }
  if constexpr (NRED == 2) reduce_dq(NJ - 1, (NJ - 1) & 1);

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
}

}  // namespace tri
