// Forward kernel: flash-style triangle attention.
//
// Work unit: (batch*head, R consecutive pair rows i, block of NW*32 queries j).
// Wave w owns one tile of 32 queries for all R rows.  The three operands of the
// iteration space (i, j, k) live in three places:
//   * bias[j, k] does not depend on the row: one packed bias tile (registers) is
//     reused by the R rows, which divides its L2 traffic by R;
//   * K[i], V[i] do not depend on the query: they are streamed through LDS in
//     tiles of BK keys (natural row-major layout, double-buffered) and shared by
//     the NW waves;
//   * Q[i, j] and the output accumulator stay in registers for the whole sweep.
// Scores are computed TRANSPOSED, S^T = K Q^T, so that a lane owns one query
// (column) and 16 keys of every 32-key tile: the softmax running reference / sum
// are per-lane scalars, and the probabilities are already in B-operand layout
// for O^T += V^T P^T, whose A operand V^T comes from the natural V tile through
// transposing LDS reads.
//
// Raw-score domain: acc = sqrt(d) * bias + q.k (the converted bias tile is the
// accumulator init of the score MFMA and is shared by the R rows);
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

template <typename T, int D, int NW, int R, int BK>
__global__ __launch_bounds__(NW * 64) void tri_fwd_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);   // MFMA steps over the head dim
  constexpr int DM = (D + 31) / 32;  // 32-row tiles of O^T
  constexpr int PS = 32 / (2 * KP);  // MFMA steps over a 32-key tile
  constexpr int KU = BK / 32;
  constexpr int NT = NW * 64;

  // One stage: K rows of the R pair rows | V rows | packed bias tiles of the NW waves.
  // Two stages (double buffer), then the keep words of the R rows.  The tiles are
  // filled by direct global->LDS loads and read through the swizzle of LdsTile.
  using Tile = LdsTile<T, D>;
  constexpr int ROWB = Tile::ROWB;
  constexpr int OFF_K = 0, OFF_V = R * BK * ROWB, OFF_B = 2 * R * BK * ROWB;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);  // one packed 32 x 32 bias tile
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
  const int jt = j_wave >> 5;

  const T* qbh = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbh = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbh = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;

  // per-row state.  A fully masked row drops the q.k and bias terms (all logits
  // equal): its Q operand is zero and it skips the bias.
  bool flagged[R];
  frag qf[R][DS];
  f32x16 oacc[R][DM];
  float mref[R], mc[R], lrun[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    flagged[r] = a.rowflag[(int64_t)b * N + i] != 0;
    for (int w = tid; w < a.nwords; w += NT) keep_s[r * a.nwords + w] = a.keep[((int64_t)b * N + i) * a.nwords + w];
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      if (j < N && !flagged[r])
        qf[r][s] = *reinterpret_cast<const frag*>(qbh + i * a.sq.i + (int64_t)j * a.sq.j + 2 * KP * s + KP * g);
      else
        qf[r][s] = E::zero();
    }
    mref[r] = kNeg;
    mc[r] = kNeg;
    lrun[r] = 0.f;
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) oacc[r][mt] = zero16();
  }

  const float c = a.c;

  // keep words of the BK keys starting at kt0 for every row; false when no row
  // attends to any of them (such stages are skipped: their probabilities are zero)
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

  // Stage loads: direct global->LDS, issued unconditionally (indices clamped into
  // range instead of branching).  A clamped key row duplicates the last valid one;
  // its keep bit is clear, so it contributes exactly zero.
  const int jt_ld = min(jt, a.NP - 1);
  auto issue_loads = [&](int kt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    Tile::template fill<R * BK, NW>(st + OFF_K, [&](int x) {
      return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sk.j; }, wave, lane);
    Tile::template fill<R * BK, NW>(st + OFF_V, [&](int x) {
      return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sv.j; }, wave, lane);
    // each wave fetches the packed bias tiles of its own query tile: 2 x 1 KiB per key tile
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const T* p = pack_bh + (((int64_t)jt_ld * a.NP + min((kt0 >> 5) + u, a.NP - 1)) * 2 * 64 + lane) * 8;
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) {
        unsigned char* dst = st + OFF_B + (wave * KU + u) * BIAS_B + r2 * (BIAS_B / 2);
        if constexpr (sizeof(T) == 2) {
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512), (TRI_L3 void*)dst, 16, 0, 0);
        } else {
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512), (TRI_L3 void*)dst, 16, 0, 0);
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512 + 4), (TRI_L3 void*)(dst + 1024), 16, 0, 0);
        }
      }
    }
  };
  // the 16 bias values of this lane for key tile u of the stage, raw-score domain
  auto bias_from_lds = [&](int buf, int u) -> f32x16 {
    const unsigned char* src = tri_smem + buf * STAGE + OFF_B + (wave * KU + u) * BIAS_B;
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

  // one stage of compute from LDS buffer `buf`
  auto compute_stage = [&](int buf, const uint32_t (*kw)[KU]) {
    const unsigned char* st = tri_smem + buf * STAGE;
    if (wave_active) {
      // The KU*R tiles of the stage run as a software pipeline inside the wave: the
      // MFMA chain that produces the scores of tile t+1 is issued before the
      // softmax arithmetic of tile t, so the matrix pipe works on t+1 while the
      // vector ALU works on t (dependent MFMAs queue in the matrix pipe without
      // holding up the wave's other instructions).  K operands are read from LDS
      // two tiles ahead, V^T operands one softmax ahead of their use.
      constexpr int TS = KU * R;
      auto k_operand = [&](int t, frag* kf) {
        const int u = t / R, r = t % R;
#pragma unroll
        for (int sd = 0; sd < DS; ++sd) kf[sd] = Tile::operand(st + OFF_K, r * BK + 32 * u + perm32(jl), sd, g);
      };
      // The bias tile does not depend on the pair row: it is converted to fp32 in
      // the raw-score domain once per stage and key tile, and then serves as the
      // accumulator init (C operand) of the first score MFMA of each of the R rows.
      f32x16 biasv[KU];
#pragma unroll
      for (int u = 0; u < KU; ++u) biasv[u] = bias_from_lds(buf, u);
      auto scores = [&](int t, const frag* kf) -> f32x16 {
        const int u = t / R, r = t % R;
        f32x16 sc;
        const bool mixed = kw[r][u] != 0xffffffffu;
        if (mixed) {
          sc = mask_tile(kw[r][u], g);
          if (!flagged[r]) {
#pragma unroll
            for (int v = 0; v < 16; ++v) sc[v] += biasv[u][v];
          }
          sc = E::mfma(kf[0], qf[r][0], sc);
        } else if (flagged[r]) {
          sc = E::mfma(kf[0], qf[r][0], zero16());
        } else {
          sc = E::mfma(kf[0], qf[r][0], biasv[u]);
        }
#pragma unroll
        for (int sd = 1; sd < DS; ++sd) sc = E::mfma(kf[sd], qf[r][sd], sc);
        return sc;
      };

      frag kf1[DS], kf2[DS];
      k_operand(0, kf1);
      if constexpr (TS > 1) k_operand(1, kf2);
      f32x16 sc = scores(0, kf1);
#pragma unroll
      for (int t = 0; t < TS; ++t) {
        const int u = t / R, r = t % R;
        f32x16 sn;
        if (t + 1 < TS) {
#pragma unroll
          for (int sd = 0; sd < DS; ++sd) kf1[sd] = kf2[sd];
          if (t + 2 < TS) k_operand(t + 2, kf2);
          sn = scores(t + 1, kf1);
        }
        if (kw[r][u] != 0) {  // a row that attends to no key of this tile adds nothing
          // V^T rows as A operand of the second product
          frag vf[DM][PS];
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
#pragma unroll
            for (int s2 = 0; s2 < PS; ++s2) vf[mt][s2] = Tile::tr_operand(st + OFF_V, r * BK + 32 * u, s2, 32 * mt, D, lane);
          // exponent arguments against the current reference; results of an fma are
          // canonical floats, so the max below needs no extra canonicalisation
          float arg[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) arg[v] = __builtin_fmaf(sc[v], c, -mc[r]);
          float amax = fmaxf(arg[0], arg[1]);
#pragma unroll
          for (int v = 2; v < 16; v += 2) amax = fmaxf(amax, fmaxf(arg[v], arg[v + 1]));
          amax = half_max(amax);
          if (__any(amax > kLazy)) {
            // some query outgrew the reference: raise it to the running maximum
            float mx = fmaxf(sc[0], sc[1]);
#pragma unroll
            for (int v = 2; v < 16; ++v) mx = fmaxf(mx, sc[v]);
            mx = half_max(mx);
            const float mnew = fmaxf(mref[r], mx);
            const float alpha = fast_exp2((mref[r] - mnew) * c);
            lrun[r] *= alpha;
#pragma unroll
            for (int mt = 0; mt < DM; ++mt)
#pragma unroll
              for (int v = 0; v < 16; ++v) oacc[r][mt][v] *= alpha;
            mref[r] = mnew;
            mc[r] = mnew * c;
#pragma unroll
            for (int v = 0; v < 16; ++v) arg[v] = __builtin_fmaf(sc[v], c, -mc[r]);
          }
          float p[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) p[v] = fast_exp2(arg[v]);
#pragma unroll
          for (int s2 = 0; s2 < PS; ++s2) {
            const frag pf = E::pack(&p[KP * s2]);
            lrun[r] = frag_sum(pf, lrun[r]);
#pragma unroll
            for (int mt = 0; mt < DM; ++mt) oacc[r][mt] = E::mfma(vf[mt][s2], pf, oacc[r][mt]);
          }
        }
        if (t + 1 < TS) sc = sn;
      }
    }

  };

  // The stage loop is unrolled by two so that the two sets of keep words swap
  // roles without being copied.
  uint32_t keep0[R][KU], keep1[R][KU];
  __syncthreads();  // keep words visible
  int kt0 = next_live(0, keep0);
  issue_loads(min(kt0, N - 1), 0);
  wait_dma();
  __syncthreads();
  while (kt0 < N) {
    // past the last live stage the prefetch re-reads a valid stage that nobody uses
    int kt1 = next_live(kt0 + BK, keep1);
    issue_loads(min(kt1, N - 1), 1);
    compute_stage(0, keep0);
    wait_dma();
    __syncthreads();
    if (kt1 >= N) break;
    kt0 = kt1;
    kt1 = next_live(kt0 + BK, keep0);
    issue_loads(min(kt1, N - 1), 0);
    compute_stage(1, keep1);
    wait_dma();
    __syncthreads();
    kt0 = kt1;
  }

  if (!wave_active) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    const float ltot = half_sum(lrun[r]);
    if (i >= N || j >= N) continue;
    T* orow = reinterpret_cast<T*>(a.o) + (((int64_t)bh * N + i) * N) * D;
    store_rows<T, D, DM>(orow + (int64_t)j * D, oacc[r], 1.0f / ltot, g);
    if (g == 0) {
      float lse = kLn2 * (mc[r] + fast_log2(ltot));
      if (flagged[r]) lse = a.neg_inf + lse;
      a.lse[((int64_t)bh * N + i) * N + j] = lse;
    }
  }
}

}  // namespace tri
