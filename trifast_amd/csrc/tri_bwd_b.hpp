// Backward kernel 3 of 3: db[j, k] = sum over rows i of dS[i, j, k].
//
// Work unit: (batch*head, block of queries j, block of keys k); the kernel walks
// all n pair rows i and keeps the db tile in fp32 registers the whole time, so
// the reduction over i has one fixed order and needs no atomics.  Per row a wave
// recomputes, for its WJ x WK tiles of 32x32,
//   S^T = K Q^T (+bias), P^T = exp2(S^T c - lse), dP^T = V dO^T, dS^T = P^T (dP^T - delta)
// with every operand in its natural row-major layout (rows of Q, dO, K, V are
// read straight from global memory as MFMA operands), and adds dS^T into db.
//
// Replaces _bwd_b of reference src/trifast/triton.py:394-501.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int WJ, int WK>
struct BRowFrags {
  using frag = typename Elem<T>::frag;
  static constexpr int DS = D / (2 * Elem<T>::KP);
  frag q[WJ][DS], dout[WJ][DS], k[WK][DS], v[WK][DS];
  float lse2[WJ], delta[WJ];
  uint32_t keepw[WK];
  bool flagged;
};

template <typename T, int D, int WJ, int WK, bool PREFETCH>
__global__ __launch_bounds__(256) void tri_bwd_b_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  using Row = BRowFrags<T, D, WJ, WK>;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int jl = lane & 31, g = lane >> 5;
  const int bh = blockIdx.z;
  const int b = bh / a.H, h = bh % a.H;
  const int N = a.N;
  // 2 x 2 waves per workgroup; they share nothing but the launch
  const int j_wave = (blockIdx.x * 2 + (wave & 1)) * (WJ * 32);
  const int k_wave = (blockIdx.y * 2 + (wave >> 1)) * (WK * 32);
  if (j_wave >= N || k_wave >= N) return;

  const T* qbase = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbase = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbase = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobase = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse_bh = a.lse + (int64_t)bh * N * N;
  const float* delta_bh = a.delta + (int64_t)bh * N * N;
  const uint32_t* keep_b = a.keep + (int64_t)b * N * a.nwords;
  const uint8_t* flag_b = a.rowflag + (int64_t)b * N;
  const float lse2_flagged = fast_log2((float)N);

  // bias tile in the raw-score domain, used as the accumulator init of every row
  f32x16 biasr[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk)
      biasr[tj][tk] = bias_tile<T>(pack_bh, a.NP, (j_wave >> 5) + tj, (k_wave >> 5) + tk, lane, a.sqrt_d, 0.f);

  f32x16 dbacc[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) dbacc[tj][tk] = zero16();

  auto load_row = [&](Row& r, int i) {
    r.flagged = flag_b[i] != 0;
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
      const int w = k_wave / 32 + tk;
      r.keepw[tk] = (w < a.nwords) ? keep_b[(int64_t)i * a.nwords + w] : 0u;
      const int key = k_wave + 32 * tk + perm32(jl);  // tile row m stands for key perm32(m)
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int dofs = 2 * KP * s + KP * g;
        if (key < N) {
          r.k[tk][s] = *reinterpret_cast<const frag*>(kbase + i * a.sk.i + (int64_t)key * a.sk.j + dofs);
          r.v[tk][s] = *reinterpret_cast<const frag*>(vbase + i * a.sv.i + (int64_t)key * a.sv.j + dofs);
        } else {
          r.k[tk][s] = E::zero();
          r.v[tk][s] = E::zero();
        }
      }
    }
#pragma unroll
    for (int tj = 0; tj < WJ; ++tj) {
      const int j = j_wave + 32 * tj + jl;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int dofs = 2 * KP * s + KP * g;
        if (j < N) {
          r.q[tj][s] = *reinterpret_cast<const frag*>(qbase + i * a.sq.i + (int64_t)j * a.sq.j + dofs);
          r.dout[tj][s] = *reinterpret_cast<const frag*>(dobase + i * a.sdo.i + (int64_t)j * a.sdo.j + dofs);
        } else {
          r.q[tj][s] = E::zero();
          r.dout[tj][s] = E::zero();
        }
      }
      if (j < N) {
        r.lse2[tj] = r.flagged ? lse2_flagged : lse_bh[(int64_t)i * N + j] * kLog2e;
        r.delta[tj] = delta_bh[(int64_t)i * N + j];
      } else {
        r.lse2[tj] = 0.f;
        r.delta[tj] = 0.f;
      }
    }
  };

  const float c = a.c;
  auto compute_row = [&](const Row& r) {
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
      if (r.keepw[tk] == 0) continue;
      const uint32_t myw = r.keepw[tk] >> (8 * g);
      const bool mixed = r.keepw[tk] != 0xffffffffu;
#pragma unroll
      for (int tj = 0; tj < WJ; ++tj) {
        f32x16 s = r.flagged ? zero16() : biasr[tj][tk];
        f32x16 dp = zero16();
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) {
          // a fully masked row ignores q.k as well as the bias
          s = E::mfma(r.k[tk][sd], r.flagged ? E::zero() : r.q[tj][sd], s);
          dp = E::mfma(r.v[tk][sd], r.dout[tj][sd], dp);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          float p = fast_exp2(__builtin_fmaf(s[v], c, -r.lse2[tj]));
          if (mixed) p = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? p : 0.f;
          dbacc[tj][tk][v] += p * (dp[v] - r.delta[tj]);
        }
      }
    }
  };

  if constexpr (PREFETCH) {
    Row cur, nxt;
    load_row(cur, 0);
    for (int i = 0; i < N; ++i) {
      if (i + 1 < N) load_row(nxt, i + 1);
      compute_row(cur);
      cur = nxt;
    }
  } else {
    Row cur;
    for (int i = 0; i < N; ++i) {
      load_row(cur, i);
      compute_row(cur);
    }
  }

  T* db_bh = reinterpret_cast<T*>(a.db) + (int64_t)bh * N * N;
  const bool vec_store = (N % 8) == 0;
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj) {
    const int j = j_wave + 32 * tj + jl;
    if (j >= N) continue;
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int key0 = k_wave + 32 * tk + 16 * r + 8 * g;
        T* dst = db_bh + (int64_t)j * N + key0;
        if (vec_store && key0 + 8 <= N) {
          if constexpr (sizeof(T) == 2) {
            typename E::vec ov;
#pragma unroll
            for (int e = 0; e < 8; ++e) ov[e] = (T)dbacc[tj][tk][8 * r + e];
            *reinterpret_cast<typename E::vec*>(dst) = ov;
          } else {
#pragma unroll
            for (int e4 = 0; e4 < 2; ++e4) {
              f32x4 ov;
#pragma unroll
              for (int e = 0; e < 4; ++e) ov[e] = dbacc[tj][tk][8 * r + 4 * e4 + e];
              *reinterpret_cast<f32x4*>(dst + 4 * e4) = ov;
            }
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (key0 + e < N) dst[e] = (T)dbacc[tj][tk][8 * r + e];
        }
      }
    }
  }
}

}  // namespace tri
