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
//   P^T = exp2(S^T c - lse*log2e),  dP^T = V dO^T,  dS^T = P^T * (dP^T - delta),
//   dq^T += K^T dS^T,               dq = dq^T / sqrt(d),
// with K^T read from the natural K tile through transposing LDS reads.
// delta is written (fp32) for the dk/dv and db kernels, so this one runs first.
//
// Replaces _bwd_q of reference src/trifast/triton.py:274-383.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int NW, int R, int BK>
__global__ __launch_bounds__(NW * 64) void tri_bwd_q_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int KU = BK / 32;
  constexpr int ROWB = Tile::ROWB;
  // one stage: K rows of the R pair rows | V rows | packed bias tiles of the NW waves
  constexpr int OFF_K = 0, OFF_V = R * BK * ROWB, OFF_B = 2 * R * BK * ROWB;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);
  constexpr int STAGE = OFF_B + NW * KU * BIAS_B;
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];
  uint32_t* keep_s = reinterpret_cast<uint32_t*>(tri_smem + 2 * STAGE);

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
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
  constexpr int NT = NW * 64;

  const T* qbh = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbh = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbh = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobh = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;

  // per-row state; a fully masked row drops the q.k and bias terms (all logits equal)
  bool flagged[R];
  frag qf[R][DS], dof[R][DS];
  float lse2[R], delta[R];
  f32x16 dqacc[R][DM];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    flagged[r] = a.rowflag[(int64_t)b * N + i] != 0;
    for (int w = tid; w < a.nwords; w += NT) keep_s[r * a.nwords + w] = a.keep[((int64_t)b * N + i) * a.nwords + w];
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
    delta[r] = dsum;
    lse2[r] = (j >= N) ? 0.f : (flagged[r] ? fast_log2((float)N) : a.lse[((int64_t)bh * N + i) * N + jc] * kLog2e);
    if (j < N && i0 + r < N && g == 0) a.delta[((int64_t)bh * N + i) * N + j] = dsum;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) dqacc[r][mt] = zero16();
  }

  const float c = a.c;

  auto stage_keep = [&](int kt0, uint32_t (*keepw)[KU]) -> bool {
    uint32_t any = 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        const int w = kt0 / 32 + u;
        keepw[r][u] = (w < a.nwords) ? keep_s[r * a.nwords + w] : 0u;
        any |= keepw[r][u];
      }
    return any != 0;
  };
  auto next_live = [&](int kt0, uint32_t (*keepw)[KU]) -> int {
    while (kt0 < N && !stage_keep(kt0, keepw)) kt0 += BK;
    return kt0;
  };

  // Stage loads: direct global->LDS, issued unconditionally with clamped indices.
  // A clamped key row duplicates the last valid one; its keep bit is clear.
  auto issue_loads = [&](int kt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    Tile::template fill<R * BK, NW>(st + OFF_K, [&](int x) {
      return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sk.j; }, wave, lane);
    Tile::template fill<R * BK, NW>(st + OFF_V, [&](int x) {
      return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sv.j; }, wave, lane);
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const T* p = pack_bh + (((int64_t)jt_ld * a.NP + min((kt0 >> 5) + u, a.NP - 1)) * 2 * 64 + lane) * 8;
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

  auto compute_stage = [&](int buf, const uint32_t (*kw)[KU]) {
    const unsigned char* st = tri_smem + buf * STAGE;
    // The KU*R tiles of the stage run as a software pipeline inside the wave: the
    // two MFMA chains (scores, dP) of tile t+1 are issued before the exponentials
    // of tile t.
    constexpr int TS = KU * R;
    f32x16 biasv[KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) biasv[u] = bias_from_lds(st, u);

    auto chains = [&](int t, f32x16& sc, f32x16& dp) {
      const int u = t / R, r = t % R;
      // key rows as A operands; tile row m stands for key perm32(m)
      const int row = r * BK + 32 * u + perm32(jl);
      if (flagged[r]) sc = zero16();
      else sc = E::mfma(Tile::operand(st + OFF_K, row, 0, g), qf[r][0], biasv[u]);
      dp = E::mfma(Tile::operand(st + OFF_V, row, 0, g), dof[r][0], zero16());
#pragma unroll
      for (int sd = 1; sd < DS; ++sd) {
        if (!flagged[r]) sc = E::mfma(Tile::operand(st + OFF_K, row, sd, g), qf[r][sd], sc);
        dp = E::mfma(Tile::operand(st + OFF_V, row, sd, g), dof[r][sd], dp);
      }
    };

    f32x16 sc, dp;
    chains(0, sc, dp);
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      const int u = t / R, r = t % R;
      f32x16 sn, dn;
      if (t + 1 < TS) chains(t + 1, sn, dn);
      if (kw[r][u] != 0) {  // a row that attends to no key of this tile has dS = 0
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = fast_exp2(__builtin_fmaf(sc[v], c, -lse2[r]));
          ds[v] = p * (dp[v] - delta[r]);
        }
        if (kw[r][u] != 0xffffffffu) {
          const uint32_t myw = kw[r][u] >> (8 * g);
#pragma unroll
          for (int v = 0; v < 16; ++v) ds[v] = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? ds[v] : 0.f;
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
            dqacc[r][mt] = E::mfma(Tile::tr_operand(st + OFF_K, r * BK + 32 * u, s2, 32 * mt, D, lane), dsf, dqacc[r][mt]);
        }
      }
      if (t + 1 < TS) { sc = sn; dp = dn; }
    }
  };

  uint32_t keep0[R][KU], keep1[R][KU];
  __syncthreads();  // keep words visible
  int kt0 = next_live(0, keep0);
  issue_loads(min(kt0, N - 1), 0);
  wait_dma();
  __syncthreads();
  while (kt0 < N) {
    int kt1 = next_live(kt0 + BK, keep1);
    issue_loads(min(kt1, N - 1), 1);
    if (wave_active) compute_stage(0, keep0);
    wait_dma();
    __syncthreads();
    if (kt1 >= N) break;
    kt0 = kt1;
    kt1 = next_live(kt0 + BK, keep0);
    issue_loads(min(kt1, N - 1), 0);
    if (wave_active) compute_stage(1, keep1);
    wait_dma();
    __syncthreads();
    kt0 = kt1;
  }

  if (!wave_active || j >= N) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    if (i >= N) continue;
    T* dqrow = reinterpret_cast<T*>(a.dq) + (((int64_t)bh * N + i) * N + j) * D;
    store_rows<T, D, DM>(dqrow, dqacc[r], a.scale, g);
  }
}

}  // namespace tri
