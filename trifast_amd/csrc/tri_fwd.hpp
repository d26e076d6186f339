// Forward kernel: flash-style triangle attention for one pair row per workgroup.
//
// Work unit: (batch*head, row i, block of NW*QT*32 queries j).  K[i] and V[i] are
// streamed through LDS in tiles of BK keys (natural row-major layout); each wave
// keeps QT tiles of 32 queries in registers.  Scores are computed TRANSPOSED,
// S^T = K Q^T, so that a lane owns one query (column) and 16 keys of every 32-key
// tile: the softmax running max / sum are per-lane scalars, and the
// probabilities are already in B-operand layout for O^T += V^T P^T, whose A
// operand V^T comes from the natural V tile through transposing LDS reads.
//
// Raw-score domain: acc = bias * sqrt(d) + q.k  (bias is the accumulator init);
// p = exp2(acc * c - ref * c) with c = log2(e) / sqrt(d).  `ref` is the running
// reference of the online softmax: it is raised to the running maximum only when
// some query of the wave exceeds it by more than kLazy (in log2 units), so the
// accumulator rescale is rare; p stays below 2^kLazy, which fp32/bf16/fp16 hold.
//
// Replaces _fwd of reference src/trifast/triton.py:19-132.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

constexpr float kLazy = 8.0f;

template <typename T, int D, int NW, int QT, int BK>
__global__ __launch_bounds__(NW * 64) void tri_fwd_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);   // MFMA steps over the head dim
  constexpr int DM = (D + 31) / 32;  // 32-row tiles of O^T
  constexpr int PS = 32 / (2 * KP);  // MFMA steps over a 32-key tile
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
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;

  // Q tiles as B operands: lane owns query j, slots 2*KP*s + KP*g .. +KP-1 of d.
  // A fully masked row drops the q.k and bias terms (all logits equal).
  frag qf[QT][DS];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int j = j_wave + 32 * t + jl;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      if (j < N && !flagged)
        qf[t][s] = *reinterpret_cast<const frag*>(qrow + (int64_t)j * a.sq.j + 2 * KP * s + KP * g);
      else
        qf[t][s] = E::zero();
    }
  }

  f32x16 oacc[QT][DM];
  float mref[QT], mc[QT], lrun[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    mref[t] = kNeg;
    mc[t] = kNeg;
    lrun[t] = 0.f;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) oacc[t][mt] = zero16();
  }

  const float c = a.c;
  const float lazy_raw = kLazy / c;
  for (int kt0 = 0; kt0 < N; kt0 += BK) {
    uint32_t keepw[KU];
    uint32_t any = 0;
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int w = kt0 / 32 + u;
      keepw[u] = (w < a.nwords) ? keep_row[w] : 0u;
      any |= keepw[u];
    }
    if (any == 0) continue;  // every key of this tile is masked or out of range

    __syncthreads();
    lds_load_natural<T, D, BK, LD, NT>(Ks, krow + (int64_t)kt0 * a.sk.j, a.sk.j, N - kt0, tid);
    lds_load_natural<T, D, BK, LD, NT>(Vs, vrow + (int64_t)kt0 * a.sv.j, a.sv.j, N - kt0, tid);
    __syncthreads();
    if (!wave_active) continue;

#pragma unroll
    for (int u = 0; u < KU; ++u) {
      if (keepw[u] == 0) continue;
      // K tile rows as A operand; tile row m stands for key perm32(m)
      frag kf[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s)
        kf[s] = *reinterpret_cast<const frag*>(&Ks[32 * u + perm32(jl)][2 * KP * s + KP * g]);
      // V^T rows as A operand of the second product
      frag vf[DM][PS];
#pragma unroll
      for (int mt = 0; mt < DM; ++mt)
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) vf[mt][s2] = tr_operand<T, LD>(Vs, 32 * u, s2, 32 * mt, D, lane);

      const uint32_t myw = keepw[u] >> (8 * g);
      const bool mixed = keepw[u] != 0xffffffffu;

#pragma unroll
      for (int t = 0; t < QT; ++t) {
        f32x16 s;
        if (!flagged)
          s = bias_tile<T>(pack_bh, a.NP, (j_wave >> 5) + t, (kt0 >> 5) + u, lane, a.sqrt_d, 0.f);
        else
          s = zero16();
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) s = E::mfma(kf[sd], qf[t][sd], s);
        if (mixed) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            s[v] = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? s[v] : kNeg;
        }
        float mx = fmaxf(s[0], s[1]);
#pragma unroll
        for (int v = 2; v < 16; v += 2) mx = fmaxf(mx, fmaxf(s[v], s[v + 1]));
        mx = half_max(mx);
        if (__any(mx > mref[t] + lazy_raw)) {
          const float mnew = fmaxf(mref[t], mx);
          const float alpha = fast_exp2((mref[t] - mnew) * c);
          lrun[t] *= alpha;
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[t][mt][v] *= alpha;
          mref[t] = mnew;
          mc[t] = mnew * c;
        }
        float p[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) p[v] = fast_exp2(__builtin_fmaf(s[v], c, -mc[t]));
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag pf = E::pack(&p[KP * s2]);
          lrun[t] = frag_sum(pf, lrun[t]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) oacc[t][mt] = E::mfma(vf[mt][s2], pf, oacc[t][mt]);
        }
      }
    }
  }

  if (!wave_active) return;
  T* orow = reinterpret_cast<T*>(a.o) + (((int64_t)bh * N + i) * N) * D;
  float* lrow = a.lse + ((int64_t)bh * N + i) * N;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const int j = j_wave + 32 * t + jl;
    const float ltot = half_sum(lrun[t]);
    if (j >= N) continue;
    store_rows<T, D, DM>(orow + (int64_t)j * D, oacc[t], 1.0f / ltot, g);
    if (g == 0) {
      float lse = kLn2 * (mc[t] + fast_log2(ltot));
      if (flagged) lse = a.neg_inf + lse;
      lrow[j] = lse;
    }
  }
}

}  // namespace tri
