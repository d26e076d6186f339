// Backward kernel 2 of 3: dk and dv.
//
// Work unit: (batch*head, R consecutive pair rows i, block of NW*32 keys).  Wave w
// owns one tile of 32 keys for all R rows: its K and V rows (B operands) and the
// dk, dv accumulators stay in registers, and the queries of the rows are streamed
// through LDS in tiles of BJ (direct global->LDS loads, double-buffered, swizzled;
// rows of Q and dO, the saved log-sum-exp and delta, and the packed bias tiles).
// Scores are computed UN-transposed here, S = Q K^T, so that a lane owns one key
// (column) and 16 queries of every 32-query tile: P and dS are then already in
// B-operand layout for the two products that contract over queries,
//   dv^T += dO^T P,   dk^T += Q^T dS,   dk = dk^T / sqrt(d),
// whose A operands dO^T, Q^T come from the natural tiles through transposing LDS
// reads.  The bias tile (fp32, raw-score domain) is converted once per stage and
// shared by the R rows as the accumulator init of the score MFMA.
//
// Replaces _bwd_kv of reference src/trifast/triton.py:143-263.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int NW, int R, int BJ, int NBUF>
__global__ __launch_bounds__(NW * 64) void tri_bwd_kv_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int JU = BJ / 32;
  constexpr int ROWB = Tile::ROWB;
  // one stage: Q rows of the R pair rows | dO rows | lse | delta | packed bias tiles
  constexpr int OFF_Q = 0, OFF_DO = R * BJ * ROWB, OFF_LSE = 2 * R * BJ * ROWB;
  constexpr int OFF_DELTA = OFF_LSE + R * BJ * 4, OFF_B = OFF_DELTA + R * BJ * 4;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);
  constexpr int STAGE = OFF_B + NW * JU * BIAS_B;
  static_assert((R * BJ) % 64 == 0, "lse/delta rows are loaded in whole waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int kl = lane & 31, g = lane >> 5;
  const int N = a.N;
  int bx, by;
  xcd_remap(gridDim.x, bx, by);
  const int i0 = by * R;
  if (i0 >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / a.H, h = bh % a.H;
  const int k_wave = bx * (NW * 32) + wave * 32;
  const int key = k_wave + kl;
  const bool wave_active = k_wave < N;
  const int kt = min(k_wave >> 5, a.NP - 1);

  const T* qbh = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbh = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbh = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobh = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packk) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse_bh = a.lse + (int64_t)bh * N * N;
  const float* delta_bh = a.delta + (int64_t)bh * N * N;

  // per-row state: K and V tiles as B operands (lane owns key k_wave + kl)
  bool flagged[R], kept[R], tile_live[R], tile_mixed[R];
  frag kf[R][DS], vf[R][DS];
  f32x16 dkacc[R][DM], dvacc[R][DM];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    flagged[r] = a.rowflag[(int64_t)b * N + i] != 0;
    const int w = k_wave >> 5;
    const uint32_t word = (wave_active && w < a.nwords) ? a.keep[((int64_t)b * N + i) * a.nwords + w] : 0u;
    tile_live[r] = word != 0;
    tile_mixed[r] = word != 0xffffffffu;
    kept[r] = (word >> kl) & 1u;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int dofs = 2 * KP * s + KP * g;
      const int kc = min(key, N - 1);
      kf[r][s] = *reinterpret_cast<const frag*>(kbh + i * a.sk.i + (int64_t)kc * a.sk.j + dofs);
      vf[r][s] = *reinterpret_cast<const frag*>(vbh + i * a.sv.i + (int64_t)kc * a.sv.j + dofs);
    }
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      dkacc[r][mt] = zero16();
      dvacc[r][mt] = zero16();
    }
  }

  // Stage loads: direct global->LDS, issued unconditionally with clamped indices.
  // A clamped query row duplicates the last valid one (with its dO, lse and
  // delta); the duplicate's P and dS are zeroed below, so queries >= N add nothing.
  auto issue_loads = [&](int jt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    Tile::template fill<R * BJ, NW>(st + OFF_Q, [&](int x) {
      return qbh + min(i0 + x / BJ, N - 1) * a.sq.i + (int64_t)min(jt0 + x % BJ, N - 1) * a.sq.j; }, wave, lane);
    Tile::template fill<R * BJ, NW>(st + OFF_DO, [&](int x) {
      return dobh + min(i0 + x / BJ, N - 1) * a.sdo.i + (int64_t)min(jt0 + x % BJ, N - 1) * a.sdo.j; }, wave, lane);
    fill_floats<R * BJ, NW>(reinterpret_cast<float*>(st + OFF_LSE), [&](int x) {
      return lse_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + min(jt0 + x % BJ, N - 1); }, wave, lane);
    fill_floats<R * BJ, NW>(reinterpret_cast<float*>(st + OFF_DELTA), [&](int x) {
      return delta_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + min(jt0 + x % BJ, N - 1); }, wave, lane);
#pragma unroll
    for (int u = 0; u < JU; ++u) {
      const T* p = pack_bh + (((int64_t)min((jt0 >> 5) + u, a.NP - 1) * a.NP + kt) * 2 * 64 + lane) * 8;
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) {
        unsigned char* dst = st + OFF_B + (wave * JU + u) * BIAS_B + r2 * (BIAS_B / 2);
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512), (TRI_L3 void*)dst, 16, 0, 0);
        if constexpr (sizeof(T) == 4)
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512 + 4), (TRI_L3 void*)(dst + 1024), 16, 0, 0);
      }
    }
  };
  auto bias_from_lds = [&](const unsigned char* st, int u) -> f32x16 {
    const unsigned char* src = st + OFF_B + (wave * JU + u) * BIAS_B;
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

  const float c = a.c;
  const float lse2_flagged = fast_log2((float)N);

  auto compute_stage = [&](int jt0, int buf) {
    const unsigned char* st = tri_smem + buf * STAGE;
    // The JU*R tiles of the stage run as a software pipeline inside the wave: the
    // two MFMA chains (scores, dP) of tile t+1 are issued before the exponentials
    // of tile t.
    constexpr int TS = JU * R;
    f32x16 biasv[JU];
#pragma unroll
    for (int u = 0; u < JU; ++u) biasv[u] = bias_from_lds(st, u);

    auto chains = [&](int t, f32x16& sc, f32x16& dp) {
      const int u = t / R, r = t % R;
      // query rows as A operands; tile row m stands for query perm32(m)
      const int row = r * BJ + 32 * u + perm32(kl);
      if (flagged[r]) sc = zero16();
      else sc = E::mfma(Tile::operand(st + OFF_Q, row, 0, g), kf[r][0], biasv[u]);
      dp = E::mfma(Tile::operand(st + OFF_DO, row, 0, g), vf[r][0], zero16());
#pragma unroll
      for (int sd = 1; sd < DS; ++sd) {
        if (!flagged[r]) sc = E::mfma(Tile::operand(st + OFF_Q, row, sd, g), kf[r][sd], sc);
        dp = E::mfma(Tile::operand(st + OFF_DO, row, sd, g), vf[r][sd], dp);
      }
    };

    f32x16 sc, dp;
    chains(0, sc, dp);
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      const int u = t / R, r = t % R;
      f32x16 sn, dn;
      if (t + 1 < TS) chains(t + 1, sn, dn);
      if (tile_live[r] && jt0 + 32 * u < N) {
        // per-query statistics of the 16 queries this lane sees: two runs of 8
        const float* lse_s = reinterpret_cast<const float*>(st + OFF_LSE) + r * BJ + 32 * u;
        const float* del_s = reinterpret_cast<const float*>(st + OFF_DELTA) + r * BJ + 32 * u;
        float p[16], ds[16];
#pragma unroll
        for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
          for (int e4 = 0; e4 < 2; ++e4) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(lse_s + 16 * r2 + 8 * g + 4 * e4);
            const f32x4 y = *reinterpret_cast<const f32x4*>(del_s + 16 * r2 + 8 * g + 4 * e4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int v = 8 * r2 + 4 * e4 + e;
              const float l2 = flagged[r] ? lse2_flagged : x[e] * kLog2e;
              p[v] = fast_exp2(__builtin_fmaf(sc[v], c, -l2));
              ds[v] = p[v] * (dp[v] + y[e]);  // the workspace holds -delta
            }
          }
        // masked keys (this lane's column) and queries past the end contribute nothing
        const bool edge = jt0 + 32 * u + 32 > N;
        if (tile_mixed[r] || edge) {
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const bool on = kept[r] && (!edge || jt0 + 32 * u + cidx(v, g) < N);
            p[v] = on ? p[v] : 0.f;
            ds[v] = on ? ds[v] : 0.f;
          }
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag pf = E::pack(&p[KP * s2]);
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) {
            dvacc[r][mt] = E::mfma(Tile::tr_operand(st + OFF_DO, r * BJ + 32 * u, s2, 32 * mt, D, lane), pf, dvacc[r][mt]);
            dkacc[r][mt] = E::mfma(Tile::tr_operand(st + OFF_Q, r * BJ + 32 * u, s2, 32 * mt, D, lane), dsf, dkacc[r][mt]);
          }
        }
      }
      if (t + 1 < TS) { sc = sn; dp = dn; }
    }
  };

  if constexpr (NBUF == 2) {
    issue_loads(0, 0);
    wait_dma();
    __syncthreads();
    for (int jt0 = 0; jt0 < N; jt0 += 2 * BJ) {
      issue_loads(min(jt0 + BJ, N - 1), 1);
      if (wave_active) compute_stage(jt0, 0);
      wait_dma();
      __syncthreads();
      if (jt0 + BJ >= N) break;
      issue_loads(min(jt0 + 2 * BJ, N - 1), 0);
      if (wave_active) compute_stage(jt0 + BJ, 1);
      wait_dma();
      __syncthreads();
    }
  } else {
    // one stage only (the double buffer does not fit in LDS): load, then compute
    for (int jt0 = 0; jt0 < N; jt0 += BJ) {
      issue_loads(jt0, 0);
      wait_dma();
      __syncthreads();
      if (wave_active) compute_stage(jt0, 0);
      __syncthreads();
    }
  }

  if (!wave_active || key >= N) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    if (i >= N) continue;
    T* dkrow = reinterpret_cast<T*>(a.dk) + (((int64_t)bh * N + i) * N + key) * D;
    T* dvrow = reinterpret_cast<T*>(a.dv) + (((int64_t)bh * N + i) * N + key) * D;
    store_rows<T, D, DM>(dkrow, dkacc[r], a.scale, g);
    store_rows<T, D, DM>(dvrow, dvacc[r], 1.0f, g);
  }
}

}  // namespace tri
