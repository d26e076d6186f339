// Backward kernel 1 of 3: delta = rowsum(o * do) and dq.
//
// Same decomposition as the forward (one pair row i and a block of queries per
// workgroup, K[i]/V[i] streamed through LDS in natural layout, transposed scores
// so a lane owns one query): P is recomputed from the saved log-sum-exp,
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

template <typename T, int D, int NW, int QT, int BK>
__global__ __launch_bounds__(NW * 64) void tri_bwd_q_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int KU = BK / 32;
  constexpr int PAD = 16 / sizeof(T);
  constexpr int LD = D + PAD;
  constexpr int NT = NW * 64;

  __shared__ __attribute__((aligned(16))) T Ks[BK][LD];
  __shared__ __attribute__((aligned(16))) T Vs[BK][LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int jl = lane & 31, g = lane >> 5;
  const int N = a.N;
  int bx, i;
  xcd_remap(gridDim.x, bx, i);
  if (i >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / a.H, h = bh % a.H;
  const int j_wave = bx * (NW * QT * 32) + wave * (QT * 32);
  const bool wave_active = j_wave < N;

  const bool flagged = a.rowflag[(int64_t)b * N + i] != 0;
  const uint32_t* keep_row = a.keep + ((int64_t)b * N + i) * a.nwords;

  const T* qrow = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h + i * a.sq.i;
  const T* krow = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h + i * a.sk.i;
  const T* vrow = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h + i * a.sv.i;
  const T* dorow = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h + i * a.sdo.i;
  const T* orow = reinterpret_cast<const T*>(a.o) + (((int64_t)bh * N + i) * N) * D;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse_row = a.lse + ((int64_t)bh * N + i) * N;
  float* delta_row = a.delta + ((int64_t)bh * N + i) * N;

  frag qf[QT][DS], dof[QT][DS];
  float lse2[QT], delta[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int j = j_wave + 32 * t + jl;
    float dsum = 0.f;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int dofs = 2 * KP * s + KP * g;
      if (j < N) {
        qf[t][s] = flagged ? E::zero() : *reinterpret_cast<const frag*>(qrow + (int64_t)j * a.sq.j + dofs);
        dof[t][s] = *reinterpret_cast<const frag*>(dorow + (int64_t)j * a.sdo.j + dofs);
        const frag of = *reinterpret_cast<const frag*>(orow + (int64_t)j * D + dofs);
        if constexpr (KP == 1) {
          dsum += (float)of * (float)dof[t][s];
        } else {
#pragma unroll
          for (int e = 0; e < KP; ++e) dsum += (float)of[e] * (float)dof[t][s][e];
        }
      } else {
        qf[t][s] = E::zero();
        dof[t][s] = E::zero();
      }
    }
    dsum = half_sum(dsum);
    delta[t] = dsum;
    if (j < N) {
      lse2[t] = flagged ? fast_log2((float)N) : lse_row[j] * kLog2e;
      if (g == 0) delta_row[j] = dsum;
    } else {
      lse2[t] = 0.f;
    }
  }

  f32x16 dqacc[QT][DM];
#pragma unroll
  for (int t = 0; t < QT; ++t)
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) dqacc[t][mt] = zero16();

  const float c = a.c;
  for (int kt0 = 0; kt0 < N; kt0 += BK) {
    uint32_t keepw[KU];
    uint32_t any = 0;
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int w = kt0 / 32 + u;
      keepw[u] = (w < a.nwords) ? keep_row[w] : 0u;
      any |= keepw[u];
    }
    if (any == 0) continue;

    __syncthreads();
    lds_load_natural<T, D, BK, LD, NT>(Ks, krow + (int64_t)kt0 * a.sk.j, a.sk.j, N - kt0, tid);
    lds_load_natural<T, D, BK, LD, NT>(Vs, vrow + (int64_t)kt0 * a.sv.j, a.sv.j, N - kt0, tid);
    __syncthreads();
    if (!wave_active) continue;

#pragma unroll
    for (int u = 0; u < KU; ++u) {
      if (keepw[u] == 0) continue;
      frag kf[DS], vf[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        kf[s] = *reinterpret_cast<const frag*>(&Ks[32 * u + perm32(jl)][2 * KP * s + KP * g]);
        vf[s] = *reinterpret_cast<const frag*>(&Vs[32 * u + perm32(jl)][2 * KP * s + KP * g]);
      }
      frag ktf[DM][PS];
#pragma unroll
      for (int mt = 0; mt < DM; ++mt)
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) ktf[mt][s2] = tr_operand<T, LD>(Ks, 32 * u, s2, 32 * mt, D, lane);

      const uint32_t myw = keepw[u] >> (8 * g);
      const bool mixed = keepw[u] != 0xffffffffu;

#pragma unroll
      for (int t = 0; t < QT; ++t) {
        f32x16 s;
        if (!flagged)
          s = bias_tile<T>(pack_bh, a.NP, (j_wave >> 5) + t, (kt0 >> 5) + u, lane, a.sqrt_d, 0.f);
        else
          s = zero16();
        f32x16 dp = zero16();
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) {
          s = E::mfma(kf[sd], qf[t][sd], s);
          dp = E::mfma(vf[sd], dof[t][sd], dp);
        }
        float ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float p = fast_exp2(__builtin_fmaf(s[v], c, -lse2[t]));
          if (mixed) p = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? p : 0.f;
          ds[v] = p * (dp[v] - delta[t]);
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) dqacc[t][mt] = E::mfma(ktf[mt][s2], dsf, dqacc[t][mt]);
        }
      }
    }
  }

  if (!wave_active) return;
  T* dqrow = reinterpret_cast<T*>(a.dq) + (((int64_t)bh * N + i) * N) * D;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int j = j_wave + 32 * t + jl;
    if (j >= N) continue;
    store_rows<T, D, DM>(dqrow + (int64_t)j * D, dqacc[t], a.scale, g);
  }
}

}  // namespace tri
