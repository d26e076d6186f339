// Backward kernel 2 of 3: dk and dv.
//
// Work unit: (batch*head, R consecutive pair rows i, block of NW*32 keys).  Wave w
// owns one tile of 32 keys for all R rows: its K and V rows (B operands) and the
// dk, dv accumulators stay in registers, and the queries of the rows are streamed
// through LDS in tiles of BJ (direct global->LDS loads, double-buffered, swizzled;
// rows of Q and dO, the lse and delta operand words left by the dq kernel, and the packed
// bias tiles).  Scores are computed UN-transposed here, S = Q K^T, so that a lane
// owns one key (column) and 16 queries of every 32-query tile: P and dS are then
// already in B-operand layout for the two products that contract over queries,
//   dv^T += dO^T P,   dk^T += Q^T dS,   dk = dk^T / sqrt(d),
// whose A operands dO^T, Q^T come from the natural tiles through transposing LDS
// reads.  The per-element additive terms ride on the matrix pipe: the bias tile
// (fp32, raw-score domain, converted once per stage and shared by the R rows) is
// the accumulator init of the score MFMA, and the per-query terms -lse*sqrt(d) and
// -delta enter through one extra MFMA each (see rank1_operand, OffsetMask), so that
// P = exp2(c * acc) and dS = P * dP' are one multiply each.  Masked keys get a large
// negative score from the MFMA that adds -lse, which makes their P and dS zero.
//
// Replaces _bwd_kv of reference src/trifast/triton.py:143-263.
#pragma once
#include <type_traits>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

// Two waves per SIMD (at most 256 registers) wherever the tile fits them or nearly
// does: a few registers over would otherwise halve the occupancy.
template <typename T, int D, int R, int BJ>
constexpr int bwd_kv_min_waves() {
  constexpr int row_bytes = D * (int)sizeof(T);
  return (row_bytes >= 512 || (row_bytes == 128 && R == 1) || (row_bytes <= 64 && R * BJ <= 64)) ? 2 : 1;
}

template <typename T, int D, int NW, int R, int BJ, int NBUF>
__global__ __launch_bounds__(NW * 64, (bwd_kv_min_waves<T, D, R, BJ>())) void tri_bwd_kv_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int DM = (D + 31) / 32;
  constexpr int PS = 32 / (2 * KP);
  constexpr int JU = BJ / 32;
  constexpr int ROWB = Tile::ROWB;
  // one stage: Q rows of the R pair rows | dO rows | lse2 | -delta | packed bias tiles
  constexpr int OFF_Q = 0, OFF_DO = R * BJ * ROWB, OFF_LSE = 2 * R * BJ * ROWB;
  constexpr int OFF_DELTA = OFF_LSE + R * BJ * 4, OFF_B = OFF_DELTA + R * BJ * 4;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);
  constexpr int STAGE = OFF_B + NW * JU * BIAS_B;
  static_assert((R * BJ) % 64 == 0, "lse/delta rows are loaded in whole waves");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  const float* lse2_bh = reinterpret_cast<const float*>(a.lse2) + (int64_t)bh * N * N;    // 32-bit words, moved as floats
  const float* delta_bh = reinterpret_cast<const float*>(a.delta) + (int64_t)bh * N * N;

  // per-row state: K and V tiles as B operands (lane owns key k_wave + kl).  A
  // fully masked row drops the q.k and bias terms from its scores: its K operand
  // is zero here (K itself is not needed for dk, dv) and it skips the bias.
  bool flagged[R], tile_live[R];
  frag kf[R][DS], vf[R][DS];
  frag keyop[R];  // ones | mask element of this lane's key: B operand of the offset-and-mask MFMA
  f32x16 dkacc[R][DM], dvacc[R][DM];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    // (wave-uniform values, pinned to scalar registers so that the branches on
    // them are real branches and not lane masks)
    flagged[r] = __builtin_amdgcn_readfirstlane(a.rowflag[(int64_t)b * N + i]) != 0;
    const int w = k_wave >> 5;
    const uint32_t word = __builtin_amdgcn_readfirstlane((wave_active && w < a.nwords) ? a.keep[((int64_t)b * N + i) * a.nwords + w] : 0u);
    tile_live[r] = word != 0;
    {
      typename OffsetMask<T>::Keys ko;
      ko.init(kl, g);
      keyop[r] = ko.masked(word);
    }
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int dofs = 2 * KP * s + KP * g;
      const int kc = min(key, N - 1);
      kf[r][s] = flagged[r] ? E::zero() : *reinterpret_cast<const frag*>(kbh + i * a.sk.i + (int64_t)kc * a.sk.j + dofs);
      vf[r][s] = *reinterpret_cast<const frag*>(vbh + i * a.sv.i + (int64_t)kc * a.sv.j + dofs);
    }
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      dkacc[r][mt] = zero16();
      dvacc[r][mt] = zero16();
    }
  }

  // lane-constant LDS offsets: Q and dO rows as natural operands (tile row m stands
  // for query perm32(m)) and again through transposing reads
  OperandOffsets<T, D> ofs;
  ofs.init(perm32(kl), lane);

  // per-lane source pointers of the stage tiles for queries 0..BJ-1
  TileStream<T, D, R * BJ, NW> qstream, dostream;
  qstream.init([&](int x) { return qbh + min(i0 + x / BJ, N - 1) * a.sq.i + (int64_t)(x % BJ) * a.sq.j; }, wave, lane);
  dostream.init([&](int x) { return dobh + min(i0 + x / BJ, N - 1) * a.sdo.i + (int64_t)(x % BJ) * a.sdo.j; }, wave, lane);
  FloatStream<R * BJ, NW> lstream, dstream;
  lstream.init([&](int x) { return lse2_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + x % BJ; }, wave, lane);
  dstream.init([&](int x) { return delta_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + x % BJ; }, wave, lane);
  const T* bias_lane = pack_bh + ((int64_t)kt * 2 * 64 + lane) * 8;

  // Stage loads: direct global->LDS.  A ragged last stage clamps query indices: a
  // clamped row duplicates the last valid one, and the compute of that stage gives
  // the duplicates P = dS = 0.
  auto issue_loads = [&](int jt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    if (jt0 + BJ <= N) {
      qstream.issue(st + OFF_Q, (int64_t)jt0 * a.sq.j, wave);
      dostream.issue(st + OFF_DO, (int64_t)jt0 * a.sdo.j, wave);
      lstream.issue(reinterpret_cast<float*>(st + OFF_LSE), jt0, wave);
      dstream.issue(reinterpret_cast<float*>(st + OFF_DELTA), jt0, wave);
    } else {
      asm volatile("" ::);  // keeps this rare path a real branch
      Tile::template fill<R * BJ, NW>(st + OFF_Q, [&](int x) {
        return qbh + min(i0 + x / BJ, N - 1) * a.sq.i + (int64_t)min(jt0 + x % BJ, N - 1) * a.sq.j; }, wave, lane);
      Tile::template fill<R * BJ, NW>(st + OFF_DO, [&](int x) {
        return dobh + min(i0 + x / BJ, N - 1) * a.sdo.i + (int64_t)min(jt0 + x % BJ, N - 1) * a.sdo.j; }, wave, lane);
      fill_floats<R * BJ, NW>(reinterpret_cast<float*>(st + OFF_LSE), [&](int x) {
        return lse2_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + min(jt0 + x % BJ, N - 1); }, wave, lane);
      fill_floats<R * BJ, NW>(reinterpret_cast<float*>(st + OFF_DELTA), [&](int x) {
        return delta_bh + (int64_t)min(i0 + x / BJ, N - 1) * N + min(jt0 + x % BJ, N - 1); }, wave, lane);
    }
#pragma unroll
    for (int u = 0; u < JU; ++u) {
      const T* p = bias_lane + (int64_t)min((jt0 >> 5) + u, a.NP - 1) * a.NP * 1024;
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
  // the per-query operand word (lse or delta term) of the query this lane's A
  // operand row stands for, in tile (r, u)
  const float c = a.c;
  typename OffsetMask<T>::Queries lseop;  // the query's -lse word | ones: A operand of that MFMA
  lseop.init(0u, g);
  auto query_word = [&](const unsigned char* st, int off, int r, int u) -> uint32_t {
    return reinterpret_cast<const uint32_t*>(st + off)[r * BJ + 32 * u + perm32(kl)];
  };

  // One stage of compute.  The JU*R tiles run as a software pipeline inside the
  // wave: the two MFMA chains (scores, dP) of tile t+1 are issued before the
  // exponentials of tile t.  EDGE stages hold queries past the end.
  // COMMON stages belong to a wave none of whose rows is fully masked or has a dead key
  // tile: the stage then has no branch, and the MFMA chains of the next tile are
  // scheduled into the vector arithmetic of the current one (branches would split them
  // into blocks of their own).
  auto compute_stage = [&](auto edge_tag, auto common_tag, int jt0, int buf) __attribute__((always_inline)) {
    constexpr bool EDGE = decltype(edge_tag)::value;
    constexpr bool COMMON = decltype(common_tag)::value && !EDGE;
    const unsigned char* st = tri_smem + buf * STAGE;
    if (!wave_active) return;
    constexpr int TS = JU * R;
    f32x16 biasv[JU];
#pragma unroll
    for (int u = 0; u < JU; ++u) biasv[u] = bias_from_lds(st, u);

    // scores: bias tile (accumulator init) - lse*sqrt(d) (per query, one MFMA) + Q K^T;
    // dP - delta: -delta (per query, one MFMA) + dO V^T
    auto chains = [&](int t, f32x16& sc, f32x16& dp) {
      const int u = t / R, r = t % R;
      const unsigned char* qt = st + OFF_Q + (r * BJ + 32 * u) * ROWB;
      const unsigned char* dot = st + OFF_DO + (r * BJ + 32 * u) * ROWB;
      uint32_t lw = query_word(st, OFF_LSE, r, u);
      if constexpr (EDGE) {
        // queries past the end: a huge lse makes their P and dS zero
        if (jt0 + 32 * u + perm32(kl) >= N) lw = split_word<T>(E::kMaskElem);
      }
      const frag ones = E::splat(1.0f);
      // -lse per query and the key mask through one MFMA (see OffsetMask; the roles of
      // the two operands are swapped here: rows are queries, columns are keys)
      lseop.set(lw, g);
      if (COMMON || !flagged[r]) {
        sc = E::mfma(lseop.get(), keyop[r], biasv[u]);
      } else {
        // rare: kept a real branch so that the common case starts from the bias
        // tile in place (a select between the two inits would copy 16 registers)
        asm volatile("" ::);
        sc = E::mfma(lseop.get(), keyop[r], zero16());
      }
      dp = E::mfma(rank1_operand<T>(query_word(st, OFF_DELTA, r, u), g), ones, zero16());
#pragma unroll
      for (int sd = 0; sd < DS; ++sd) {
        sc = E::mfma(ofs.natural(qt, sd), kf[r][sd], sc);
        dp = E::mfma(ofs.natural(dot, sd), vf[r][sd], dp);
      }
    };

    f32x16 sc, dp;
    chains(0, sc, dp);
#pragma unroll
    for (int t = 0; t < TS; ++t) {
      const int u = t / R, r = t % R;
      f32x16 sn, dn;
      if (t + 1 < TS) chains(t + 1, sn, dn);
      if (COMMON || (tile_live[r] && (!EDGE || jt0 + 32 * u < N))) {
        float p[16], ds[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          p[v] = fast_exp2(sc[v] * c);
          ds[v] = p[v] * dp[v];
        }
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          const frag pf = E::pack(&p[KP * s2]);
          const frag dsf = E::pack(&ds[KP * s2]);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) {
            dvacc[r][mt] = E::mfma(ofs.transposed(st + OFF_DO + (r * BJ + 32 * u) * ROWB, s2, mt), pf, dvacc[r][mt]);
            dkacc[r][mt] = E::mfma(ofs.transposed(st + OFF_Q + (r * BJ + 32 * u) * ROWB, s2, mt), dsf, dkacc[r][mt]);
          }
        }
      }
      if (t + 1 < TS) { sc = sn; dp = dn; }
    }
  };

  // Stages that lie inside the query range run in the main loop; a ragged last
  // stage runs after it with the edge handling.
  const int nfull = N / BJ;  // whole stages
  const bool ragged = N % BJ != 0;
  if constexpr (NBUF == 2) {
    issue_loads(0, 0);
    wait_dma();
    __syncthreads();
    // (the whole loop exists twice; a wave picks its version once.  Both run the same
    // stages and barriers.)
    auto whole_stages = [&](auto common_tag) __attribute__((always_inline)) {
      int s = 0;
      for (; s + 1 < nfull; s += 2) {
        issue_loads((s + 1) * BJ, 1);
        compute_stage(std::false_type{}, common_tag, s * BJ, 0);
        wait_dma();
        __syncthreads();
        if ((s + 2) * BJ < N) issue_loads((s + 2) * BJ, 0);
        compute_stage(std::false_type{}, common_tag, (s + 1) * BJ, 1);
        wait_dma();
        __syncthreads();
      }
      return s;
    };
    bool common = wave_active;
#pragma unroll
    for (int r = 0; r < R; ++r) common = common && !flagged[r] && tile_live[r];
    const int s = common ? whole_stages(std::true_type{}) : whole_stages(std::false_type{});
    // buffer 0 now holds stage s: the last whole one, the ragged one, or a spare
    if (s < nfull) {
      if (ragged) issue_loads((s + 1) * BJ, 1);
      compute_stage(std::false_type{}, std::false_type{}, s * BJ, 0);
      if (ragged) {
        wait_dma();
        __syncthreads();
        compute_stage(std::true_type{}, std::false_type{}, (s + 1) * BJ, 1);
      }
    } else if (ragged) {
      compute_stage(std::true_type{}, std::false_type{}, s * BJ, 0);
    }
  } else {
    // one stage only (the double buffer does not fit in LDS): load, then compute
    for (int s = 0; s < nfull; ++s) {
      issue_loads(s * BJ, 0);
      wait_dma();
      __syncthreads();
      compute_stage(std::false_type{}, std::false_type{}, s * BJ, 0);
      __syncthreads();
    }
    if (ragged) {
      issue_loads(nfull * BJ, 0);
      wait_dma();
      __syncthreads();
      compute_stage(std::true_type{}, std::false_type{}, nfull * BJ, 0);
    }
  }

  if (!wave_active) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    if (i >= N) continue;
    T* dkrow = reinterpret_cast<T*>(a.dk) + b * a.sdk.b + h * a.sdk.h + i * a.sdk.i + key * a.sdk.j;
    T* dvrow = reinterpret_cast<T*>(a.dv) + b * a.sdv.b + h * a.sdv.h + i * a.sdv.i + key * a.sdv.j;
    store_rows_any<T, D, DM>(dkrow, dkacc[r], a.scale, g, key < N);
    store_rows_any<T, D, DM>(dvrow, dvacc[r], 1.0f, g, key < N);
  }
}

}  // namespace tri
