// Forward kernel: flash-style triangle attention for one pair row per workgroup.
//
// Work unit: (batch*head, row i, block of NW*QT*32 queries j).  K[i] and V[i] are
// streamed through LDS in tiles of BK keys; each wave keeps QT tiles of 32
// queries in registers.  Scores are computed TRANSPOSED, S^T = K Q^T, so that a
// lane owns one query (column) and 16 keys of every 32-key tile: the softmax
// running max / sum are per-lane scalars, and the probabilities are already in
// B-operand layout for O^T += V^T P^T.
//
// Raw-score domain: acc = bias * sqrt(d) + q.k  (bias is the accumulator init);
// p = exp2(acc * c - max * c) with c = log2(e) / sqrt(d).
//
// Replaces _fwd of reference src/trifast/triton.py:19-132.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"

namespace tri {

// Cooperative load of a [ROWS x D] row-major tile (row stride `stride` elements,
// rows >= nrows read as zero) into LDS in natural layout.
template <typename T, int D, int ROWS, int LD, int NT>
TRI_DEV void lds_load_natural(T (*dst)[LD], const T* src, int64_t stride, int nrows, int tid) {
  using E = Elem<T>;
  constexpr int VEC = E::VEC;
  constexpr int CPR = D / VEC;  // 16-byte chunks per row
  for (int c = tid; c < ROWS * CPR; c += NT) {
    const int row = c / CPR, col = (c % CPR) * VEC;
    typename E::vec val;
    if (row < nrows) {
      val = *reinterpret_cast<const typename E::vec*>(src + (int64_t)row * stride + col);
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) val[e] = (T)0.f;
    }
    *reinterpret_cast<typename E::vec*>(&dst[row][col]) = val;
  }
}

// Cooperative load of a [ROWS x D] row-major tile into LDS TRANSPOSED:
// dst[d][row].  16-bit types pack two adjacent rows into one 32-bit store.
template <typename T, int D, int ROWS, int LD, int NT>
TRI_DEV void lds_load_transposed(T (*dst)[LD], const T* src, int64_t stride, int nrows, int tid) {
  using E = Elem<T>;
  constexpr int VEC = E::VEC;
  constexpr int CPR = D / VEC;
  if constexpr (sizeof(T) == 2) {
    typedef T t2 __attribute__((ext_vector_type(2)));
    constexpr int PAIRS = ROWS / 2;
    for (int c = tid; c < PAIRS * CPR; c += NT) {
      const int pr = c % PAIRS, col = (c / PAIRS) * VEC;
      const int r0 = 2 * pr, r1 = 2 * pr + 1;
      typename E::vec a, b;
#pragma unroll
      for (int e = 0; e < VEC; ++e) { a[e] = (T)0.f; b[e] = (T)0.f; }
      if (r0 < nrows) a = *reinterpret_cast<const typename E::vec*>(src + (int64_t)r0 * stride + col);
      if (r1 < nrows) b = *reinterpret_cast<const typename E::vec*>(src + (int64_t)r1 * stride + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        t2 w;
        w[0] = a[e];
        w[1] = b[e];
        *reinterpret_cast<t2*>(&dst[col + e][r0]) = w;
      }
    }
  } else {
    for (int c = tid; c < ROWS * CPR; c += NT) {
      const int row = c % ROWS, col = (c / ROWS) * VEC;
      typename E::vec a;
#pragma unroll
      for (int e = 0; e < VEC; ++e) a[e] = (T)0.f;
      if (row < nrows) a = *reinterpret_cast<const typename E::vec*>(src + (int64_t)row * stride + col);
#pragma unroll
      for (int e = 0; e < VEC; ++e) dst[col + e][row] = a[e];
    }
  }
}

// 8 consecutive bias values bias_row[key0 .. key0+7] as floats (0 outside [0, N)).
template <typename T>
TRI_DEV void load_bias8(const T* bias_row, int key0, int N, bool row_ok, bool vec_ok, float* out) {
  if (row_ok && vec_ok && key0 + 8 <= N) {
    if constexpr (sizeof(T) == 2) {
      typename Elem<T>::vec x = *reinterpret_cast<const typename Elem<T>::vec*>(bias_row + key0);
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = (float)x[e];
    } else {
      f32x4 x0 = *reinterpret_cast<const f32x4*>(bias_row + key0);
      f32x4 x1 = *reinterpret_cast<const f32x4*>(bias_row + key0 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { out[e] = x0[e]; out[4 + e] = x1[e]; }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      out[e] = (row_ok && key0 + e < N) ? (float)bias_row[key0 + e] : 0.f;
  }
}

template <typename T, int D, int NW, int QT, int BK>
__global__ __launch_bounds__(NW * 64) void tri_fwd_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);   // MFMA steps over the head dim
  constexpr int DM = (D + 31) / 32;  // 32-row tiles of O^T
  constexpr int DROWS = DM * 32;
  constexpr int PS = 32 / (2 * KP);  // MFMA steps over a 32-key tile
  constexpr int KU = BK / 32;
  constexpr int PAD = 16 / sizeof(T);
  constexpr int NT = NW * 64;

  __shared__ __attribute__((aligned(16))) T Ks[BK][D + PAD];
  __shared__ __attribute__((aligned(16))) T Vt[DROWS][BK + PAD];

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
  const T* bias_bh = reinterpret_cast<const T*>(a.bias) + b * a.sbias.b + h * a.sbias.h;

  if constexpr (DROWS > D) {  // zero the padding rows of V^T once
    for (int c = tid; c < (DROWS - D) * (BK + PAD); c += NT)
      Vt[D + c / (BK + PAD)][c % (BK + PAD)] = (T)0.f;
  }

  // Q tiles as B operands: lane owns query j, slots 2*KP*s + KP*g .. +KP-1 of d.
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
  float mrun[QT], lrun[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    mrun[t] = kNeg;
    lrun[t] = 0.f;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) oacc[t][mt] = zero16();
  }

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
    if (any == 0) continue;  // every key of this tile is masked or out of range

    __syncthreads();
    lds_load_natural<T, D, BK, D + PAD, NT>(Ks, krow + (int64_t)kt0 * a.sk.j, a.sk.j, N - kt0, tid);
    lds_load_transposed<T, D, BK, BK + PAD, NT>(Vt, vrow + (int64_t)kt0 * a.sv.j, a.sv.j, N - kt0, tid);
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
        for (int s2 = 0; s2 < PS; ++s2)
          vf[mt][s2] = *reinterpret_cast<const frag*>(&Vt[32 * mt + jl][32 * u + cidx(KP * s2, g)]);

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
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) s = E::mfma(kf[sd], qf[t][sd], s);
        if (mixed) {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            s[v] = ((myw >> (16 * (v / 8) + (v % 8))) & 1u) ? s[v] : kNeg;
        }
        float mx = s[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) mx = fmaxf(mx, s[v]);
        mx = fmaxf(mx, xhalf(mx));
        const float mnew = fmaxf(mrun[t], mx);
        const float alpha = fast_exp2((mrun[t] - mnew) * c);
        const float mc = mnew * c;
        float p[16];
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[v] = fast_exp2(__builtin_fmaf(s[v], c, -mc));
          psum += p[v];
        }
        lrun[t] = lrun[t] * alpha + psum;
        mrun[t] = mnew;
#pragma unroll
        for (int mt = 0; mt < DM; ++mt)
#pragma unroll
          for (int v = 0; v < 16; ++v) oacc[t][mt][v] *= alpha;
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag pf = E::pack(&p[KP * s2]);
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
    const float ltot = lrun[t] + xhalf(lrun[t]);
    if (j >= N) continue;
    const float inv = 1.0f / ltot;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int d0 = 32 * mt + 8 * a4 + 4 * g;
        if (d0 < D) {
          typename E::vec4 ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = (T)(oacc[t][mt][4 * a4 + e] * inv);
          *reinterpret_cast<typename E::vec4*>(orow + (int64_t)j * D + d0) = ov;
        }
      }
    }
    if (g == 0) {
      float lse = kLn2 * (mrun[t] * c + fast_log2(ltot));
      if (flagged) lse = a.neg_inf + lse;
      lrow[j] = lse;
    }
  }
}

}  // namespace tri
