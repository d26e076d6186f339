// Backward kernel 1 of 3: delta = rowsum(o * do) and dq.
//
// Same decomposition as the forward: (batch*head, R consecutive pair rows i, block
// of NW*32 queries).  Wave w owns one tile of 32 queries for all R rows (Q, dO
// operands, lse, delta and the dq accumulator in registers); K[i] and V[i] are
// streamed through LDS in tiles of BK keys (direct global->LDS loads,
// double-buffered, swizzled) together with the packed bias tiles, and the bias
// tile (fp32, raw-score domain) is shared by the R rows as the accumulator init of
// the score MFMA.  With transposed scores (a lane owns one query) P is recomputed
// from the saved log-sum-exp,
//   P^T = exp2(S^T c - lse*log2e),  dP^T - delta = V dO^T - delta,  dS^T = P^T * (dP^T - delta),
//   dq^T += K^T dS^T,               dq = dq^T / sqrt(d),
// with K^T read from the natural K tile through transposing LDS reads.  -delta is
// the accumulator init of the dP MFMA (16 registers per row that never change),
// so the subtraction costs nothing.  Masked keys get a large negative score
// through one extra MFMA (see OffsetMask), which makes their P and dS zero.
//
// This kernel runs first: it writes -delta and -lse*sqrt(d) (ln n for lse in fully
// masked rows) per query, as rank-1 MFMA operand words, for the dk/dv and db kernels.
//
// Replaces _bwd_q of reference src/trifast/triton.py:274-383.
#pragma once
#include <type_traits>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int NW, int R, int BK>
__global__ __launch_bounds__(NW * 64, (R >= 4) ? 1 : 2) void tri_bwd_q_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int KU = BK / 32;
  constexpr int ROWB = Tile::ROWB;
  // one stage: K rows of the R pair rows | V rows | packed bias tiles of the NW waves;
  // two stages, then the key-tile bitmaps
  constexpr int OFF_K = 0, OFF_V = R * BK * ROWB, OFF_B = 2 * R * BK * ROWB;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);
  constexpr int OFF_KW = OFF_B + NW * KU * BIAS_B;  // keep words of the stage's tiles, [R][KU] (64 slots)
  constexpr int STAGE = OFF_KW + 256;
  static_assert(R * KU <= 64, "the keep words of a stage are one 64-lane load");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int jl = lane & 31, g = lane >> 5;
  const int N = a.N;
  int bx, by;
  xcd_remap(gridDim.x, bx, by);
  const int i0 = by * R;
  if (i0 >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / a.H, h = bh % a.H;
  const int j_wave = bx * (NW * 32) + wave * 32;
  const int j = j_wave + jl;
  const bool wave_active = j_wave < N;
  const int jt_ld = min(j_wave >> 5, a.NP - 1);

  const T* qbh = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbh = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbh = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobh = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;

  // per-row state; a fully masked row drops the q.k and bias terms (all logits equal)
  bool flagged[R];
  bool any_flagged = false;
  const uint32_t* keep_row[R];
  frag qf[R][DS], dof[R][DS];
  float lse2[R];
  f32x16 ndelta[R];  // -delta in all 16 slots: accumulator init of the dP MFMA
  f32x16 dqacc[R][DM];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    flagged[r] = __builtin_amdgcn_readfirstlane(a.rowflag[(int64_t)b * N + i]) != 0;  // pinned to a scalar register
    any_flagged |= flagged[r];
    keep_row[r] = a.keep + ((int64_t)b * N + i) * a.nwords;
    const int jc = min(j, N - 1);
    const T* orow = reinterpret_cast<const T*>(a.o) + (((int64_t)bh * N + i) * N + jc) * D;
    float dsum = 0.f;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int dofs = 2 * KP * s + KP * g;
      qf[r][s] = (flagged[r] || j >= N) ? E::zero() : *reinterpret_cast<const frag*>(qbh + i * a.sq.i + (int64_t)jc * a.sq.j + dofs);
      dof[r][s] = (j >= N) ? E::zero() : *reinterpret_cast<const frag*>(dobh + i * a.sdo.i + (int64_t)jc * a.sdo.j + dofs);
      const frag of = *reinterpret_cast<const frag*>(orow + dofs);
      if constexpr (KP == 1) {
        dsum += (float)of * (float)dof[r][s];
      } else {
#pragma unroll
        for (int e = 0; e < KP; ++e) dsum += (float)of[e] * (float)dof[r][s][e];
      }
    }
    dsum = half_sum(dsum);
    lse2[r] = (j >= N) ? 0.f : (flagged[r] ? fast_log2((float)N) : a.lse[((int64_t)bh * N + i) * N + jc] * kLog2e);
    if (j < N && i0 + r < N && g == 0) {
      // the per-query terms of the other two backward kernels, as rank-1 MFMA operand words
      a.delta[((int64_t)bh * N + i) * N + j] = split_word<T>(-dsum);
      a.lse2[((int64_t)bh * N + i) * N + j] = split_word<T>(-lse2[r] * (kLn2 * a.sqrt_d));
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) ndelta[r][v] = -dsum;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) dqacc[r][mt] = zero16();
  }
  const float c = a.c;

  // the key mask enters the scores through one extra MFMA: keys operand with the mask
  // element of this lane's key (patched in place per tile) against a constant queries
  // operand (see OffsetMask; its per-query offset is not used here: the word is zero)
  typename OffsetMask<T>::Keys kop;
  kop.init(perm32(jl), g);
  frag qzero;
  {
    typename OffsetMask<T>::Queries qz;
    qz.init(split_word<T>(0.f), g);
    qzero = qz.get();
  }

  KeyTileMasks masks;
  masks.build<R, NW>(reinterpret_cast<uint64_t*>(tri_smem + 2 * STAGE), [&](int r) { return keep_row[r]; }, a.nwords, any_flagged, wave, lane);

  // lane-constant LDS offsets: K and V rows as natural operands (tile row m stands
  // for key perm32(m)), K rows again through transposing reads for dq
  OperandOffsets<T, D> ofs;
  ofs.init(perm32(jl), lane);

  TileStream<T, D, R * BK, NW> kstream, vstream;
  kstream.init([&](int x) { return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)(x % BK) * a.sk.j; }, wave, lane);
  vstream.init([&](int x) { return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)(x % BK) * a.sv.j; }, wave, lane);

  // Stage loads: direct global->LDS; a ragged last stage clamps key indices (the
  // duplicated rows have clear keep bits)
  const T* bias_lane = pack_bh + ((int64_t)jt_ld * a.NP * 2 * 64 + lane) * 8;
  // keep words travel with the stage (lane x of wave 0: row x / KU, key tile x % KU);
  // workgroups that attend to every key do not need them
  const uint32_t* kw_lane = a.keep + ((int64_t)b * N + min(i0 + (lane % (R * KU)) / KU, N - 1)) * a.nwords;
  const int kw_u = lane % KU;
  bool want_keep_words = true;
  auto issue_loads = [&](int kt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    if (want_keep_words && wave == 0)
      __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(kw_lane + min((kt0 >> 5) + kw_u, a.nwords - 1)), (TRI_L3 void*)(st + OFF_KW), 4, 0, 0);
    if (kt0 + BK <= N) {
      kstream.issue(st + OFF_K, (int64_t)kt0 * a.sk.j, wave);
      vstream.issue(st + OFF_V, (int64_t)kt0 * a.sv.j, wave);
    } else {
      asm volatile("" ::);  // keeps this rare path a real branch (no speculation into the common one)
      Tile::template fill<R * BK, NW>(st + OFF_K, [&](int x) {
        return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sk.j; }, wave, lane);
      Tile::template fill<R * BK, NW>(st + OFF_V, [&](int x) {
        return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sv.j; }, wave, lane);
    }
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const T* p = bias_lane + (int64_t)min((kt0 >> 5) + u, a.NP - 1) * 1024;
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) {
        unsigned char* dst = st + OFF_B + (wave * KU + u) * BIAS_B + r2 * (BIAS_B / 2);
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512), (TRI_L3 void*)dst, 16, 0, 0);
        if constexpr (sizeof(T) == 4)
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512 + 4), (TRI_L3 void*)(dst + 1024), 16, 0, 0);
      }
    }
  };
  auto bias_from_lds = [&](const unsigned char* st, int u) -> f32x16 {
    const unsigned char* src = st + OFF_B + (wave * KU + u) * BIAS_B;
    f32x16 bv;
#pragma unroll
    for (int r2 = 0; r2 < 2; ++r2) {
      if constexpr (sizeof(T) == 2) {
        const typename E::vec x = *reinterpret_cast<const typename E::vec*>(src + r2 * (BIAS_B / 2) + lane * 16);
#pragma unroll
        for (int e = 0; e < 8; ++e) bv[8 * r2 + e] = (float)x[e] * a.sqrt_d;
      } else {
        const f32x4 x0 = *reinterpret_cast<const f32x4*>(src + r2 * (BIAS_B / 2) + lane * 16);
        const f32x4 x1 = *reinterpret_cast<const f32x4*>(src + r2 * (BIAS_B / 2) + 1024 + lane * 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) { bv[8 * r2 + e] = x0[e] * a.sqrt_d; bv[8 * r2 + 4 + e] = x1[e] * a.sqrt_d; }
      }
    }
    return bv;
  };

  // One stage of compute from LDS buffer `buf`, keys kt0 .. kt0+BK-1.  The KU*R
  // tiles run as a software pipeline inside the wave: the two MFMA chains (scores,
  // dP) of tile t+1 are issued before the exponentials of tile t.
  auto compute_stage = [&](auto mode_tag, int kt0, int buf) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool PLAIN = MODE == kPlain;
    const unsigned char* st = tri_smem + buf * STAGE;
    if (!wave_active) return;
    constexpr int TS = KU * R;
    uint32_t kw[R][KU];
    if constexpr (!PLAIN) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < KU; ++u) {
          const int w = (kt0 >> 5) + u;
          kw[r][u] = __builtin_amdgcn_readfirstlane((w < a.nwords) ? reinterpret_cast<const uint32_t*>(st + OFF_KW)[r * KU + u] : 0u);
        }
    }
    f32x16 biasv[KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) biasv[u] = bias_from_lds(st, u);

    auto chains = [&](int t, f32x16& sc, f32x16& dp) {
      const int u = t / R, r = t % R;
      const unsigned char* kt = st + OFF_K + (r * BK + 32 * u) * ROWB;
      const unsigned char* vt = st + OFF_V + (r * BK + 32 * u) * ROWB;
      if constexpr (PLAIN) {
        sc = E::mfma(ofs.natural(kt, 0), qf[r][0], biasv[u]);
      } else {
        // Each case ends in the MFMA that defines sc, so that the bias tile is used
        // in place as an accumulator init (a select between inits copies 16 registers).
        if (MODE == kMasked) {
          // no fully masked row in the workgroup: the mask MFMA runs for every tile
          // (its operand is zero where nothing is masked) and nothing branches
          sc = E::mfma(ofs.natural(kt, 0), qf[r][0], E::mfma(kop.masked(kw[r][u]), qzero, biasv[u]));
        } else if (!flagged[r]) {
          if (kw[r][u] != 0xffffffffu)
            sc = E::mfma(ofs.natural(kt, 0), qf[r][0], E::mfma(kop.masked(kw[r][u]), qzero, biasv[u]));
          else
            sc = E::mfma(ofs.natural(kt, 0), qf[r][0], biasv[u]);
        } else {
          // a fully masked row has no bias (and a zero Q), but keys past the end of a
          // ragged last tile stay masked for it too
          asm volatile("" ::);
          sc = E::mfma(kop.masked(kw[r][u]), qzero, zero16());
          sc = E::mfma(ofs.natural(kt, 0), qf[r][0], sc);
        }
      }
      dp = E::mfma(ofs.natural(vt, 0), dof[r][0], ndelta[r]);
#pragma unroll
      for (int sd = 1; sd < DS; ++sd) {
        sc = E::mfma(ofs.natural(kt, sd), qf[r][sd], sc);
        dp = E::mfma(ofs.natural(vt, sd), dof[r][sd], dp);
      }
    };

    f32x16 sc, dp;
    chains(0, sc, dp);
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      const int u = t / R, r = t % R;
      f32x16 sn, dn;
      if (t + 1 < TS) chains(t + 1, sn, dn);
      bool tile_on = true;  // a row that attends to no key of this tile has dS = 0
      if constexpr (!PLAIN) tile_on = kw[r][u] != 0;
      if (tile_on) {
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = fast_exp2(__builtin_fmaf(sc[v], c, -lse2[r]));
          ds[v] = p * dp[v];
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
            dqacc[r][mt] = E::mfma(ofs.transposed(st + OFF_K + (r * BK + 32 * u) * ROWB, s2, mt), dsf, dqacc[r][mt]);
        }
      }
      if (t + 1 < TS) { sc = sn; dp = dn; }
    }
  };

  // Stage loop over the live stages, unrolled by two for the two LDS buffers; a
  // workgroup whose rows attend to every key runs the loop specialised for it.
  __syncthreads();  // key-tile bitmaps visible
  const int ntiles = a.nwords;
  auto stage_loop = [&](auto mode_tag) __attribute__((always_inline)) {
    constexpr bool PLAIN = decltype(mode_tag)::value == kPlain;
    want_keep_words = !PLAIN;
    auto next = [&](int t) { return PLAIN ? min(t, ntiles) : masks.next_live<KU>(t); };
    int t0 = next(0);
    issue_loads(min(32 * t0, N - 1), 0);
    wait_dma();
    __syncthreads();
    while (t0 < ntiles) {
      const int t1 = next(t0 + KU);
      issue_loads(min(32 * t1, N - 1), 1);
      compute_stage(mode_tag, 32 * t0, 0);
      wait_dma();
      __syncthreads();
      if (t1 >= ntiles) break;
      t0 = next(t1 + KU);
      issue_loads(min(32 * t0, N - 1), 0);
      compute_stage(mode_tag, 32 * t1, 1);
      wait_dma();
      __syncthreads();
    }
  };
  // (a last stage with fewer than KU key tiles is not plain: its missing tiles are masked)
  if (masks.all_plain() && ntiles % KU == 0) stage_loop(std::integral_constant<int, kPlain>{});
  else if (!any_flagged) stage_loop(std::integral_constant<int, kMasked>{});
  else stage_loop(std::integral_constant<int, kGeneral>{});

  if (!wave_active) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    if (i >= N) continue;
    T* dqrow = reinterpret_cast<T*>(a.dq) + b * a.sdq.b + h * a.sdq.h + i * a.sdq.i + j * a.sdq.j;
    store_rows_any<T, D, DM>(dqrow, dqacc[r], a.scale, g, j < N);
  }
}

}  // namespace tri
