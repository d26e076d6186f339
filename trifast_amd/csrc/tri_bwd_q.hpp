// Backward kernel 1 of 3: delta = rowsum(o * do) and dq.
//
// Same decomposition as the forward (one pair row i and a block of queries per
// workgroup, K[i]/V[i] streamed through LDS, transposed scores so a lane owns one
// query): P is recomputed from the saved log-sum-exp,
//   P^T = exp2(S^T c - lse*log2e),  dP^T = V dO^T,  dS^T = P^T * (dP^T - delta),
//   dq^T += K^T dS^T,               dq = dq^T / sqrt(d).
// delta is written (fp32) for the dk/dv and db kernels, so this one runs first.
//
// Replaces _bwd_q of reference src/trifast/triton.py:274-383.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_fwd.hpp"

namespace tri {

template <typename T, int D, int NW, int QT, int BK>
__global__ __launch_bounds__(NW * 64) void tri_bwd_q_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int DROWS = DM * 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int KU = BK / 32;
  constexpr int PAD = 16 / sizeof(T);
  constexpr int NT = NW * 64;

  __shared__ __attribute__((aligned(16))) T Ks[BK][D + PAD];
  __shared__ __attribute__((aligned(16))) T Vs[BK][D + PAD];
  // fp32 operands are single elements, so Ks serves the transposed reads too
  constexpr bool kTr = KP > 1;
  constexpr int TROWS = kTr ? DROWS : 1, TLD = kTr ? BK + PAD : 4;
  __shared__ __attribute__((aligned(16))) T Kt[TROWS][TLD];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int jl = lane & 31, g = lane >> 5;
  const int bh = blockIdx.z, i = blockIdx.y;
  const int b = bh / a.H, h = bh % a.H;
  const int N = a.N;
  const int j_wave = blockIdx.x * (NW * QT * 32) + wave * (QT * 32);
  const bool wave_active = j_wave < N;

  const bool flagged = a.rowflag[(int64_t)b * N + i] != 0;
  const uint32_t* keep_row = a.keep + ((int64_t)b * N + i) * a.nwords;

  const T* qrow = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h + i * a.sq.i;
  const T* krow = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h + i * a.sk.i;
  const T* vrow = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h + i * a.sv.i;
  const T* dorow = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h + i * a.sdo.i;
  const T* orow = reinterpret_cast<const T*>(a.o) + (((int64_t)bh * N + i) * N) * D;
  const T* bias_bh = reinterpret_cast<const T*>(a.bias) + b * a.sbias.b + h * a.sbias.h;
  const float* lse_row = a.lse + ((int64_t)bh * N + i) * N;
  float* delta_row = a.delta + ((int64_t)bh * N + i) * N;

  if constexpr (kTr && DROWS > D) {
    for (int c = tid; c < (DROWS - D) * (BK + PAD); c += NT)
      Kt[D + c / (BK + PAD)][c % (BK + PAD)] = (T)0.f;
  }

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
    dsum += xhalf(dsum);
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
    lds_load_natural<T, D, BK, D + PAD, NT>(Ks, krow + (int64_t)kt0 * a.sk.j, a.sk.j, N - kt0, tid);
    lds_load_natural<T, D, BK, D + PAD, NT>(Vs, vrow + (int64_t)kt0 * a.sv.j, a.sv.j, N - kt0, tid);
    if constexpr (kTr)
      lds_load_transposed<T, D, BK, TLD, NT>(Kt, krow + (int64_t)kt0 * a.sk.j, a.sk.j, N - kt0, tid);
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
        for (int s2 = 0; s2 < PS; ++s2)
          if constexpr (kTr)
            ktf[mt][s2] = *reinterpret_cast<const frag*>(&Kt[32 * mt + jl][32 * u + cidx(KP * s2, g)]);
          else
            ktf[mt][s2] = (32 * mt + jl < D) ? *reinterpret_cast<const frag*>(&Ks[32 * u + cidx(s2, g)][32 * mt + jl]) : E::zero();

      const uint32_t myw = keepw[u] >> (8 * g);
      const bool mixed = keepw[u] != 0xffffffffu;

#pragma unroll
      for (int t = 0; t < QT; ++t) {
        const int j = j_wave + 32 * t + jl;
        f32x16 s;
        if (!flagged) {
          float bv[16];
          const T* brow = bias_bh + (int64_t)j * a.sbias.j;
          load_bias8<T>(brow, kt0 + 32 * u + 8 * g, N, j < N, a.bias_vec_ok, bv);
          load_bias8<T>(brow, kt0 + 32 * u + 16 + 8 * g, N, j < N, a.bias_vec_ok, bv + 8);
#pragma unroll
          for (int v = 0; v < 16; ++v) s[v] = bv[v] * a.sqrt_d;
        } else {
          s = zero16();
        }
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
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d0 = 32 * mt + 8 * a4 + 4 * g;
        if (d0 < D) {
          typename E::vec4 ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = (T)(dqacc[t][mt][4 * a4 + e] * a.scale);
          *reinterpret_cast<typename E::vec4*>(dqrow + (int64_t)j * D + d0) = ov;
        }
      }
    }
  }
}

}  // namespace tri
