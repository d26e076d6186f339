// Forward kernel: flash-style triangle attention.
//
// Work unit: (batch*head, R consecutive pair rows i, block of NW*32 queries j).
// Wave w owns one tile of 32 queries for all R rows.  The three operands of the
// iteration space (i, j, k) live in three places:
//   * bias[j, k] does not depend on the row: one packed bias tile (registers) is
//     reused by the R rows, which divides its L2 traffic by R;
//   * K[i], V[i] do not depend on the query: they are streamed through LDS in
//     tiles of BK keys (direct global->LDS loads, swizzled, double-buffered) and
//     shared by the NW waves;
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
// the probabilities of some query of the wave sum to more than 2^kLazy within a
// tile, so the accumulator rescale is rare and no maximum is searched otherwise;
// p stays below 2^kLazy, which fp32/bf16/fp16 hold.
//
// Masks: a bitmap over the key tiles says which stages are live (others are
// skipped) and whether all of them are plain (every row attends to every key:
// the workgroup then runs a loop with no mask work and no per-tile branch).
// Otherwise a masked key gets a large negative score through one extra MFMA
// (see OffsetMask).
//
// Replaces _fwd of reference src/trifast/triton.py:19-132.
#pragma once
#include <type_traits>

#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

constexpr float kLazy = 8.0f;
constexpr float kLazyLimit = 256.0f;  // 2^kLazy

template <typename T, int D, int NW, int R, int BK>
__global__ __launch_bounds__(NW * 64, (R * (BK / 32) >= 8) ? 1 : 2) void tri_fwd_kernel(const FwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);   // MFMA steps over the head dim
  constexpr int DM = (D + 31) / 32;  // 32-row tiles of O^T
  constexpr int PS = 32 / (2 * KP);  // MFMA steps over a 32-key tile
  constexpr int KU = BK / 32;

  // One stage: K rows of the R pair rows | V rows | packed bias tiles of the NW waves.
  // Two stages (double buffer), then the key-tile bitmaps.
  using Tile = LdsTile<T, D>;
  constexpr int ROWB = Tile::ROWB;
  constexpr int OFF_K = 0, OFF_V = R * BK * ROWB, OFF_B = 2 * R * BK * ROWB;
  constexpr int BIAS_B = 2 * 64 * 8 * (int)sizeof(T);  // one packed 32 x 32 bias tile
  constexpr int OFF_KW = OFF_B + NW * KU * BIAS_B;  // keep words of the stage's tiles, [R][KU] (64 slots)
  constexpr int STAGE = OFF_KW + 256;
  static_assert(R * KU <= 64, "the keep words of a stage are one 64-lane load");
  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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
  bool any_flagged = false;
  const uint32_t* keep_row[R];
  frag qf[R][DS];
  f32x16 oacc[R][DM];
  float mref[R], mc[R], lrun[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = min(i0 + r, N - 1);  // rows past the end repeat the last one and are not stored
    flagged[r] = __builtin_amdgcn_readfirstlane(a.rowflag[(int64_t)b * N + i]) != 0;  // pinned to a scalar register
    any_flagged |= flagged[r];
    keep_row[r] = a.keep + ((int64_t)b * N + i) * a.nwords;
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

  // the key mask enters the scores through one extra MFMA: keys operand with the mask
  // element of this lane's key (patched in place per tile) against a constant queries
  // operand (see OffsetMask; its per-query offset is not used here: the word is zero)
  typename OffsetMask<T>::Keys kop;
  kop.init(perm32(jl), g);
  frag qzero;
  {
    typename OffsetMask<T>::Queries qz;
    qz.init(split_word<T>(0.f), g);
    qzero = qz.get();
  }

  KeyTileMasks masks;
  masks.build<R, NW>(reinterpret_cast<uint64_t*>(tri_smem + 2 * STAGE), [&](int r) { return keep_row[r]; }, a.nwords, any_flagged, wave, lane);

  // lane-constant LDS offsets of the operand reads: K rows as natural operands
  // (tile row m stands for key perm32(m)), V rows through transposing reads
  OperandOffsets<T, D> ofs;
  ofs.init(perm32(jl), lane);

  // per-lane source pointers of the K and V stage tiles for keys 0..BK-1
  TileStream<T, D, R * BK, NW> kstream, vstream;
  kstream.init([&](int x) { return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)(x % BK) * a.sk.j; }, wave, lane);
  vstream.init([&](int x) { return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)(x % BK) * a.sv.j; }, wave, lane);

  // Stage loads: direct global->LDS.  A stage that lies inside the key range adds
  // one uniform offset to the precomputed pointers; the last, ragged one clamps
  // key indices instead of branching (a clamped key row duplicates the last valid
  // one; its keep bit is clear, so it contributes exactly zero).
  const int jt_ld = min(jt, a.NP - 1);
  const T* bias_lane = pack_bh + ((int64_t)jt_ld * a.NP * 2 * 64 + lane) * 8;
  // keep words travel with the stage (lane x of wave 0: row x / KU, key tile x % KU);
  // workgroups that attend to every key do not need them
  const uint32_t* kw_lane = a.keep + ((int64_t)b * N + min(i0 + (lane % (R * KU)) / KU, N - 1)) * a.nwords;
  const int kw_u = lane % KU;
  bool want_keep_words = true;
  auto issue_loads = [&](int kt0, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    if (want_keep_words && wave == 0)
      __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(kw_lane + min((kt0 >> 5) + kw_u, a.nwords - 1)), (TRI_L3 void*)(st + OFF_KW), 4, 0, 0);
    if (kt0 + BK <= N) {
      kstream.issue(st + OFF_K, (int64_t)kt0 * a.sk.j, wave);
      vstream.issue(st + OFF_V, (int64_t)kt0 * a.sv.j, wave);
    } else {
      asm volatile("" ::);  // keeps this rare path a real branch (no speculation into the common one)
      Tile::template fill<R * BK, NW>(st + OFF_K, [&](int x) {
        return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sk.j; }, wave, lane);
      Tile::template fill<R * BK, NW>(st + OFF_V, [&](int x) {
        return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)min(kt0 + x % BK, N - 1) * a.sv.j; }, wave, lane);
    }
    // each wave fetches the packed bias tiles of its own query tile: 2 x 1 KiB per key tile
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const T* p = bias_lane + (int64_t)min((kt0 >> 5) + u, a.NP - 1) * 1024;
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2) {
        unsigned char* dst = st + OFF_B + (wave * KU + u) * BIAS_B + r2 * (BIAS_B / 2);
        __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512), (TRI_L3 void*)dst, 16, 0, 0);
        if constexpr (sizeof(T) == 4)
          __builtin_amdgcn_global_load_lds((const TRI_G1 void*)(p + r2 * 512 + 4), (TRI_L3 void*)(dst + 1024), 16, 0, 0);
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

  // One stage of compute from LDS buffer `buf`, keys kt0 .. kt0+BK-1.
  //
  // The KU*R tiles of the stage run as a software pipeline inside the wave: the
  // MFMA chain that produces the scores of tile t+1 is issued before the softmax
  // arithmetic of tile t, so the matrix pipe works on t+1 while the vector ALU
  // works on t.  K operands are read from LDS two tiles ahead.
  //
  // Softmax of a tile: p = exp2(acc * c - ref * c) is computed against the current
  // reference without looking for the maximum first; only when the rounded
  // probabilities of some query sum to more than 2^kLazy (which includes the
  // overflow to +inf of a query that outgrew the reference by a lot, and the very
  // first tile, whose reference is -1e30) is the reference raised to the running
  // maximum and the tile recomputed.
  auto compute_stage = [&](auto mode_tag, int kt0, int buf) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool PLAIN = MODE == kPlain;
    const unsigned char* st = tri_smem + buf * STAGE;
    if (!wave_active) return;
    constexpr int TS = KU * R;
    // keep words of the stage's tiles (wave-uniform loads)
    uint32_t kw[R][KU];
    if constexpr (!PLAIN) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int u = 0; u < KU; ++u) {
          const int w = (kt0 >> 5) + u;
          kw[r][u] = __builtin_amdgcn_readfirstlane((w < a.nwords) ? reinterpret_cast<const uint32_t*>(st + OFF_KW)[r * KU + u] : 0u);
        }
    }
    auto k_operand = [&](int t, frag* kf) {
      const int u = t / R, r = t % R;
#pragma unroll
      for (int sd = 0; sd < DS; ++sd) kf[sd] = ofs.natural(st + OFF_K + (r * BK + 32 * u) * ROWB, sd);
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
      if constexpr (PLAIN) {
        sc = E::mfma(kf[0], qf[r][0], biasv[u]);
      } else {
        // Each case ends in the MFMA that defines sc, so that the bias tile is used
        // in place as an accumulator init (a select between inits copies 16 registers).
        if (MODE == kMasked) {
          // no fully masked row in the workgroup: the mask MFMA runs for every tile
          // (its operand is zero where nothing is masked) and nothing branches
          sc = E::mfma(kf[0], qf[r][0], E::mfma(kop.masked(kw[r][u]), qzero, biasv[u]));
        } else if (!flagged[r]) {
          if (kw[r][u] != 0xffffffffu)
            sc = E::mfma(kf[0], qf[r][0], E::mfma(kop.masked(kw[r][u]), qzero, biasv[u]));
          else
            sc = E::mfma(kf[0], qf[r][0], biasv[u]);
        } else {
          // a fully masked row has no bias (and a zero Q: all its scores are equal),
          // but keys past the end of a ragged last tile stay masked for it too
          asm volatile("" ::);
          sc = E::mfma(kop.masked(kw[r][u]), qzero, zero16());
          sc = E::mfma(kf[0], qf[r][0], sc);
        }
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
      bool tile_on = true;  // a row that attends to no key of this tile adds nothing
      if constexpr (!PLAIN) tile_on = kw[r][u] != 0;
      if (tile_on) {
        // V^T rows as A operand of the second product
        frag vf[DM][PS];
#pragma unroll
        for (int mt = 0; mt < DM; ++mt)
#pragma unroll
          for (int s2 = 0; s2 < PS; ++s2) vf[mt][s2] = ofs.transposed(st + OFF_V + (r * BK + 32 * u) * ROWB, s2, mt);
        frag pf[PS];
        float ts = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2) {
          float p[KP];
#pragma unroll
          for (int e = 0; e < KP; ++e) p[e] = fast_exp2(__builtin_fmaf(sc[KP * s2 + e], c, -mc[r]));
          pf[s2] = E::pack(p);
          ts = frag_sum(pf[s2], ts);
        }
        if (__any(!(ts <= kLazyLimit))) {
          // some query outgrew the reference: raise it to the running maximum.
          // (The empty volatile asm keeps the compiler from executing this rare
          // path speculatively in line with the common one.)
          asm volatile("" ::);
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
          ts = 0.f;
#pragma unroll
          for (int s2 = 0; s2 < PS; ++s2) {
            float p[KP];
#pragma unroll
            for (int e = 0; e < KP; ++e) p[e] = fast_exp2(__builtin_fmaf(sc[KP * s2 + e], c, -mc[r]));
            pf[s2] = E::pack(p);
            ts = frag_sum(pf[s2], ts);
          }
        }
        lrun[r] += ts;
#pragma unroll
        for (int s2 = 0; s2 < PS; ++s2)
#pragma unroll
          for (int mt = 0; mt < DM; ++mt) oacc[r][mt] = E::mfma(vf[mt][s2], pf[s2], oacc[r][mt]);
      }
      if (t + 1 < TS) sc = sn;
    }
  };
  // Stage loop over the live stages, unrolled by two for the two LDS buffers.  A
  // workgroup whose rows attend to every key runs the loop specialised for plain
  // stages; any other one runs the general loop for all of its stages (mixing the
  // two inside one loop would copy the accumulators where the versions meet).
  __syncthreads();  // key-tile bitmaps visible
  const int ntiles = a.nwords;
  auto stage_loop = [&](auto mode_tag) __attribute__((always_inline)) {
    constexpr bool PLAIN = decltype(mode_tag)::value == kPlain;
    want_keep_words = !PLAIN;
    auto next = [&](int t) { return PLAIN ? min(t, ntiles) : masks.next_live<KU>(t); };
    int t0 = next(0);
    issue_loads(min(32 * t0, N - 1), 0);
    wait_dma();
    __syncthreads();
    while (t0 < ntiles) {
      // past the last live stage the prefetch re-reads a valid stage that nobody uses
      const int t1 = next(t0 + KU);
      issue_loads(min(32 * t1, N - 1), 1);
      compute_stage(mode_tag, 32 * t0, 0);
      wait_dma();
      __syncthreads();
      if (t1 >= ntiles) break;
      t0 = next(t1 + KU);
      issue_loads(min(32 * t0, N - 1), 0);
      compute_stage(mode_tag, 32 * t1, 1);
      wait_dma();
      __syncthreads();
    }
  };
  // (a last stage with fewer than KU key tiles is not plain: its missing tiles are masked)
  if (masks.all_plain() && ntiles % KU == 0) stage_loop(std::integral_constant<int, kPlain>{});
  else if (!any_flagged) stage_loop(std::integral_constant<int, kMasked>{});
  else stage_loop(std::integral_constant<int, kGeneral>{});

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
