// Backward kernel 2 of 3: dk and dv.
//
// Work unit: (batch*head, row i, block of NW*KT*32 keys).  Each wave keeps KT
// tiles of 32 keys (K and V rows as B operands) in registers and streams the
// queries of the row through LDS in tiles of BJ (natural layout).  Scores are
// computed UN-transposed here, S = Q K^T, so that a lane owns one key (column)
// and 16 queries of every 32-query tile: P and dS are then already in B-operand
// layout for the two products that contract over queries,
//   dv^T += dO^T P,   dk^T += Q^T dS,   dk = dk^T / sqrt(d),
// whose A operands dO^T, Q^T come from the natural tiles through transposing LDS
// reads.  The key mask is a per-lane constant folded into the bias conversion.
//
// Replaces _bwd_kv of reference src/trifast/triton.py:143-263.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int NW, int KT, int BJ>
__global__ __launch_bounds__(NW * 64) void tri_bwd_kv_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int JU = BJ / 32;
  constexpr int PAD = 16 / sizeof(T);
  constexpr int LD = D + PAD;
  constexpr int NT = NW * 64;

  __shared__ __attribute__((aligned(16))) T Qs[BJ][LD];
  __shared__ __attribute__((aligned(16))) T dOs[BJ][LD];
  __shared__ __attribute__((aligned(16))) float lse2s[BJ];
  __shared__ __attribute__((aligned(16))) float deltas[BJ];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int kl = lane & 31, g = lane >> 5;
  const int N = a.N;
  int bx, i;
  xcd_remap(gridDim.x, bx, i);
  if (i >= N) return;
  const int bh = blockIdx.z;
  const int b = bh / a.H, h = bh % a.H;
  const int k_wave = bx * (NW * KT * 32) + wave * (KT * 32);
  const bool wave_active = k_wave < N;

  const bool flagged = a.rowflag[(int64_t)b * N + i] != 0;
  const uint32_t* keep_row = a.keep + ((int64_t)b * N + i) * a.nwords;

  const T* qrow = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h + i * a.sq.i;
  const T* krow = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h + i * a.sk.i;
  const T* vrow = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h + i * a.sv.i;
  const T* dorow = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h + i * a.sdo.i;
  const T* pack_bh = reinterpret_cast<const T*>(a.packk) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse_row = a.lse + ((int64_t)bh * N + i) * N;
  const float* delta_row = a.delta + ((int64_t)bh * N + i) * N;

  // K and V tiles as B operands: lane owns key k_wave + 32 t + kl
  frag kf[KT][DS], vf[KT][DS];
  float lanebias[KT];   // 0 for an attended key, kNeg for a masked / out-of-range one
  bool tile_live[KT];
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int key = k_wave + 32 * t + kl;
    const int w = (k_wave + 32 * t) / 32;
    const uint32_t word = (w < a.nwords) ? keep_row[w] : 0u;
    tile_live[t] = word != 0;
    lanebias[t] = ((word >> kl) & 1u) ? 0.f : kNeg;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int dofs = 2 * KP * s + KP * g;
      if (key < N) {
        kf[t][s] = *reinterpret_cast<const frag*>(krow + (int64_t)key * a.sk.j + dofs);
        vf[t][s] = *reinterpret_cast<const frag*>(vrow + (int64_t)key * a.sv.j + dofs);
      } else {
        kf[t][s] = E::zero();
        vf[t][s] = E::zero();
      }
    }
  }

  f32x16 dkacc[KT][DM], dvacc[KT][DM];
#pragma unroll
  for (int t = 0; t < KT; ++t)
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      dkacc[t][mt] = zero16();
      dvacc[t][mt] = zero16();
    }

  const float c = a.c;
  const float lse2_flagged = fast_log2((float)N);
  for (int jt0 = 0; jt0 < N; jt0 += BJ) {
    __syncthreads();
    lds_load_natural<T, D, BJ, LD, NT>(Qs, qrow + (int64_t)jt0 * a.sq.j, a.sq.j, N - jt0, tid);
    lds_load_natural<T, D, BJ, LD, NT>(dOs, dorow + (int64_t)jt0 * a.sdo.j, a.sdo.j, N - jt0, tid);
    for (int x = tid; x < BJ; x += NT) {
      const int j = jt0 + x;
      lse2s[x] = (j < N) ? (flagged ? lse2_flagged : lse_row[j] * kLog2e) : 0.f;
      deltas[x] = (j < N) ? delta_row[j] : 0.f;
    }
    __syncthreads();
    if (!wave_active) continue;

#pragma unroll
    for (int u = 0; u < JU; ++u) {
      if (jt0 + 32 * u >= N) continue;
      // query rows as A operands; tile row m stands for query perm32(m)
      frag qa[DS], doa[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        qa[s] = flagged ? E::zero()
                        : *reinterpret_cast<const frag*>(&Qs[32 * u + perm32(kl)][2 * KP * s + KP * g]);
        doa[s] = *reinterpret_cast<const frag*>(&dOs[32 * u + perm32(kl)][2 * KP * s + KP * g]);
      }
      frag qtf[DM][PS], dotf[DM][PS];
#pragma unroll
      for (int mt = 0; mt < DM; ++mt)
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          qtf[mt][s2] = tr_operand<T, LD>(Qs, 32 * u, s2, 32 * mt, D, lane);
          dotf[mt][s2] = tr_operand<T, LD>(dOs, 32 * u, s2, 32 * mt, D, lane);
        }
      // per-query statistics of the 16 queries this lane sees: two runs of 8
      float l2[16], dl[16];
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int e4 = 0; e4 < 2; ++e4) {
          const f32x4 x = *reinterpret_cast<const f32x4*>(&lse2s[32 * u + 16 * r + 8 * g + 4 * e4]);
          const f32x4 y = *reinterpret_cast<const f32x4*>(&deltas[32 * u + 16 * r + 8 * g + 4 * e4]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            l2[8 * r + 4 * e4 + e] = x[e];
            dl[8 * r + 4 * e4 + e] = y[e];
          }
        }

#pragma unroll
      for (int t = 0; t < KT; ++t) {
        if (!tile_live[t]) continue;
        f32x16 s;
        if (!flagged) {
          s = bias_tile<T>(pack_bh, a.NP, (jt0 >> 5) + u, (k_wave >> 5) + t, lane, a.sqrt_d, lanebias[t]);
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v) s[v] = lanebias[t];
        }
        f32x16 dp = zero16();
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) {
          s = E::mfma(qa[sd], kf[t][sd], s);
          dp = E::mfma(doa[sd], vf[t][sd], dp);
        }
        float p[16], ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[v] = fast_exp2(__builtin_fmaf(s[v], c, -l2[v]));
          ds[v] = p[v] * (dp[v] - dl[v]);
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag pf = E::pack(&p[KP * s2]);
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) {
            dvacc[t][mt] = E::mfma(dotf[mt][s2], pf, dvacc[t][mt]);
            dkacc[t][mt] = E::mfma(qtf[mt][s2], dsf, dkacc[t][mt]);
          }
        }
      }
    }
  }

  if (!wave_active) return;
  T* dkrow = reinterpret_cast<T*>(a.dk) + (((int64_t)bh * N + i) * N) * D;
  T* dvrow = reinterpret_cast<T*>(a.dv) + (((int64_t)bh * N + i) * N) * D;
#pragma unroll
  for (int t = 0; t < KT; ++t) {
    const int key = k_wave + 32 * t + kl;
    if (key >= N) continue;
    store_rows<T, D, DM>(dkrow + (int64_t)key * D, dkacc[t], a.scale, g);
    store_rows<T, D, DM>(dvrow + (int64_t)key * D, dvacc[t], 1.0f, g);
  }
}

}  // namespace tri
