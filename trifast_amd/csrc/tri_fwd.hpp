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
// (see OffsetMask).  The scheduled loop further down exists in both forms; workgroups with
// a fully masked row, ragged n and fp32 take the general stage loop.
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

// BKF: keys per stage of the general stage loop, plus kFwdFast when the workgroup may take
// the scheduled loop below for rows without masked keys.
constexpr int kFwdFast = 256;
// LDS bytes of the two loops (without the key-tile bitmaps that follow them)
constexpr int fwd_stage_bytes(int D, int es, int NW, int R, int BK) { return (2 * R * BK * D + NW * (BK / 32) * 1024) * es + 256; }
// stages of the scheduled loop's ring: what is in use, what the next barrier publishes, and
// the rest in flight (four pair rows per stage leave room for three stages at two workgroups
// per compute unit; their loads are then issued three tiles before the barrier that needs them)
constexpr int fwd_fast_stages(int R) { return R >= 4 ? 3 : 4; }
constexpr int fwd_fast_stage_bytes(int D, int es, int NW, int R) { return 2 * R * 32 * D * es + NW * 2048; }
constexpr int fwd_main_lds_bytes(int D, int es, int NW, int R, int BKF) {
  const int gen = 2 * fwd_stage_bytes(D, es, NW, R, BKF % kFwdFast);
  const int fast = BKF >= kFwdFast ? fwd_fast_stages(R) * fwd_fast_stage_bytes(D, es, NW, R) : 0;
  return gen > fast ? gen : fast;
}

template <typename T, int D, int NW, int R, int BKF>
__global__ __launch_bounds__(NW * 64, (R * ((BKF % kFwdFast) / 32) >= 8) ? 1 : 2) void tri_fwd_kernel(const FwdArgs a) {
  constexpr int BK = BKF % kFwdFast;
  constexpr bool FAST = BKF >= kFwdFast;
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
  static_assert(STAGE == fwd_stage_bytes(D, (int)sizeof(T), NW, R, BK), "the launcher sizes LDS with fwd_stage_bytes");
  constexpr int LDS_MAIN = fwd_main_lds_bytes(D, (int)sizeof(T), NW, R, BKF);  // the key-tile bitmaps follow
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
  frag qzero;

  KeyTileMasks masks;
  masks.build<R, NW>(reinterpret_cast<uint64_t*>(tri_smem + LDS_MAIN), [&](int r) { return keep_row[r]; }, a.nwords, any_flagged, wave, lane);

  // lane-constant LDS offsets of the operand reads: K rows as natural operands
  // (tile row m stands for key perm32(m)), V rows through transposing reads
  OperandOffsets<T, D> ofs;
  ofs.init(perm32(jl), lane);

  // per-lane source pointers of the K and V stage tiles for keys 0..BK-1
  // (set up by the general stage loop only: the scheduled loop below has no use for them, and
  // what is live across the choice between the two loops takes registers from both)
  TileStream<T, D, R * BK, NW> kstream, vstream;
  auto setup_general = [&] {
    kop.init(perm32(jl), g);
    typename OffsetMask<T>::Queries qz;
    qz.init(split_word<T>(0.f), g);
    qzero = qz.get();
    kstream.init([&](int x) { return kbh + min(i0 + x / BK, N - 1) * a.sk.i + (int64_t)(x % BK) * a.sk.j; }, wave, lane);
    vstream.init([&](int x) { return vbh + min(i0 + x / BK, N - 1) * a.sv.i + (int64_t)(x % BK) * a.sv.j; }, wave, lane);
  };

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
  // ---- the scheduled loop: workgroups without a fully masked row, n a multiple of 32 ----------
  // Same work as the plain stage loop above, laid out as the schedule it should run in.  A
  // wave issues in order, so everything a tile needs is asked for a whole tile ahead:
  //   * a ring of three or four 32-key stages (K rows, V rows and the waves' packed bias
  //     tiles), filled by global->LDS loads that are issued two or three stages ahead; one barrier per stage, before
  //     its last tile, publishes the next stage.  Every load in the loop is an asm statement
  //     and every wait for them is a counted one written here: a load the compiler knows of
  //     (or a register it reloads from scratch) would make it wait for everything in flight;
  //   * in the slot of tile t the wave reads the K operand of tile t+1 and the V operand of
  //     tile t from LDS, issues the P.V MFMAs of tile t-1 and the score MFMAs of tile t+1,
  //     and spreads the softmax arithmetic of tile t (in units of two scores: two fma, two
  //     exp2, a packed conversion and a row-sum step) between them;
  //   * the bias tile of the next stage enters through the matrix pipe in the last slot of a
  //     stage: its packed words are the B operand against a constant A operand that holds
  //     sqrt(d) where the contraction slot is the row's key (sqrt(32) as hi + lo parts), and
  //     the product is the accumulator init of the score MFMAs of the R rows.
  // masked_tag: the rows have masked keys (none of them is fully masked): every tile takes one
  // more MFMA, which gives the masked keys a large negative score, and the stages after the
  // last one with an attended key are left out
  auto fast_loop = [&](auto masked_tag) __attribute__((always_inline)) {
    static_assert(!FAST || (sizeof(T) == 2 && BK == 32 && R >= 2), "16-bit types, 32-key stages, two or more pair rows");
    if constexpr (FAST) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
    typedef T pair_t __attribute__((ext_vector_type(2)));
    constexpr int NS = fwd_fast_stages(R);
    constexpr int FSTAGE = fwd_fast_stage_bytes(D, (int)sizeof(T), NW, R);
    constexpr int FOFF_V = R * 32 * ROWB, FOFF_B = 2 * R * 32 * ROWB;
    constexpr int G = 2 * R * 32 * Tile::CPR / 64;  // 1 KiB wave loads per stage: K rows, then V rows
    static_assert(G % NW == 0, "every wave issues the same number of loads");
    constexpr int XN = G / NW;
    constexpr int NLD = XN + 2;  // loads per wave and stage: its share of K and V, its bias tile
    auto SB = [] { __builtin_amdgcn_sched_barrier(0); };
    const int ns = MASKED ? masks.last_live() : N >> 5;
    // the keep words of the stage in use and of the next one, one per pair row (wave-uniform:
    // scalar loads, issued a stage ahead of their use)
    uint32_t kwc[R], kwn[R];
    auto fetch_keep_words = [&](int stage, uint32_t* kw) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < R; ++r) kw[r] = MASKED ? uniform_word(keep_row[r], min(stage, a.nwords - 1)) : 0xffffffffu;
    };
    if constexpr (MASKED) {
      kop.init(perm32(jl), g);
      typename OffsetMask<T>::Queries qz;
      qz.init(split_word<T>(0.f), g);
      qzero = qz.get();
      fetch_keep_words(0, kwc);
      fetch_keep_words(1, kwn);
    }

    // this wave's loads of a stage: a 32-bit byte offset per lane from the stage's first K / V row
    uint32_t lofs[XN];
#pragma unroll
    for (int x = 0; x < XN; ++x) {
      const int gi = x * NW + wave;
      const bool is_k = gi < G / 2;
      const int p = (gi % (G / 2)) * 64 + lane;
      const int r_ = p / Tile::CPR, cc = (p % Tile::CPR) ^ Tile::swz(r_);
      const int64_t rr = min(i0 + r_ / 32, N - 1) - i0;
      const Str5& st = is_k ? a.sk : a.sv;
      lofs[x] = (uint32_t)((rr * st.i + (int64_t)(r_ % 32) * st.j + cc * Tile::VEC) * (int64_t)sizeof(T));
    }
    const uint32_t lane16 = (uint32_t)lane * 16u;
    const T* krow0 = kbh + (int64_t)i0 * a.sk.i;
    const T* vrow0 = vbh + (int64_t)i0 * a.sv.i;
    const T* bias_wave = pack_bh + (int64_t)jt_ld * a.NP * 1024;  // packed bias tiles of this wave's queries
    const uint32_t lds0 = (uint32_t)(uintptr_t)(TRI_L3 unsigned char*)tri_smem;
    // (the sources move along the keys by a constant step per stage: three scalar pointers)
    const int64_t kstep = 32 * a.sk.j, vstep = 32 * a.sv.j;
    const T* kfill = krow0;
    const T* vfill = vrow0;
    const T* bfill = bias_wave;
    int filled = 0;  // the stage the pointers stand at
    auto issue_fast = [&](int boff) {
#pragma unroll
      for (int x = 0; x < XN; ++x) {
        const int gi = x * NW + wave;
        const T* base = gi < G / 2 ? kfill : vfill;  // wave-uniform
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(boff + gi * 1024));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(lofs[x]), "s"(base) : "memory", "m0");
      }
      const uint32_t dstb = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(boff + FOFF_B + wave * 2048));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024" : : "s"(dstb), "v"(lane16), "s"(bfill) : "memory", "m0");
      // (the second load lands 1 KiB further: the instruction offset applies to both addresses)
      // past the last stage the pointers stay: a valid stage is fetched again, which nobody uses
      const bool more = filled + 1 < ns;
      kfill += more ? kstep : 0;
      vfill += more ? vstep : 0;
      bfill += more ? 1024 : 0;
      filled += 1;
    };
    // A operand of the bias products: row m of the score tile stands for key perm32(m); half r2
    // of the packed words gives the contraction slots 8 g + e the keys 16 r2 + 8 g + e
    constexpr int NPART = D == 32 ? 2 : 1;
    constexpr int NB = 2 * NPART;
    frag bsel[2][NPART];
    {
      const T hi = (T)a.sqrt_d;
      const T part[2] = {hi, (T)(a.sqrt_d - (float)hi)};
#pragma unroll
      for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
        for (int pp = 0; pp < NPART; ++pp) {
          const int e = perm32(jl) - 16 * r2 - 8 * g;
          const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, part[pp]) << (16 * (e & 1));
          u32x4v w;
#pragma unroll
          for (int x = 0; x < 4; ++x) w[x] = (e >= 0 && e < 8 && (e >> 1) == x) ? bits : 0u;
          asm volatile("" : "+v"(w));  // resident: not rebuilt from the lane id at every use
          bsel[r2][pp] = __builtin_bit_cast(frag, w);
        }
    }
    const pair_t ones = {(T)1.0f, (T)1.0f};

    // absolute LDS addresses of this lane's operand reads in the stage in use (K rows as natural
    // operands, V rows through transposing reads, the wave's bias words); they move with the ring
    uint32_t ak[DS], avl[DM], avh[DM], ab;
#pragma unroll
    for (int sd = 0; sd < DS; ++sd) ak[sd] = lds0 + (uint32_t)ofs.nat[sd];
#pragma unroll
    for (int mt = 0; mt < DM; ++mt) {
      avl[mt] = lds0 + (uint32_t)(FOFF_V + ofs.tlo[mt]);
      avh[mt] = lds0 + (uint32_t)(FOFF_V + ofs.thi[mt]);
    }
    ab = lds0 + (uint32_t)(FOFF_B + wave * 2048) + lane16;
    auto lds_frag = [](uint32_t addr) { return *reinterpret_cast<TRI_L3 const frag*>((uintptr_t)addr); };
    auto lds_tr = [](uint32_t lo, uint32_t hi) {
      const auto x = lds_tr4(reinterpret_cast<TRI_L3 const T*>((uintptr_t)lo));
      const auto y = lds_tr4(reinterpret_cast<TRI_L3 const T*>((uintptr_t)hi));
      frag f;
#pragma unroll
      for (int e = 0; e < 4; ++e) { f[e] = x[e]; f[4 + e] = y[e]; }
      return f;
    };

    // ---- the state that moves from slot to slot ----
    f32x16 sc_cur = zero16(), bias_s = zero16();
    frag vf_prev[DM][PS], pf_prev[PS];
#pragma unroll
    for (int s2 = 0; s2 < PS; ++s2) {
      pf_prev[s2] = E::zero();
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) vf_prev[mt][s2] = E::zero();
    }

    // ---- prologue: the first stages on their way, bias tile and scores of the first tile ----
#pragma unroll
    for (int st = 0; st < NS - 1; ++st) issue_fast(st * FSTAGE);
    // (a wait the compiler knows: the loads made before the loop, the Q operands among them, no
    // longer count as in flight, or it would wait for everything again where the loop first
    // uses them, in every trip)
    wait_dma_known();
    ring_sync<0>();
    if (wave_active) {
#pragma unroll
      for (int x = 0; x < NB; ++x)
        bias_s = E::mfma(bsel[x / NPART][x % NPART], lds_frag(ab + (x / NPART) * 1024), bias_s);
      sc_cur = bias_s;
      if constexpr (MASKED) sc_cur = E::mfma(kop.masked(kwc[0]), qzero, sc_cur);
#pragma unroll
      for (int sd = 0; sd < DS; ++sd) sc_cur = E::mfma(lds_frag(ak[sd]), qf[0][sd], sc_cur);
    }

    enum { F_B, F_PV, F_S, F_M };
    // (the loop exists twice: for waves with queries, and for the waves past the end of the pair
    // row, which only take part in the loads and barriers; one loop with the test inside would
    // make the compiler copy the state where the two cases meet)
    auto stage_loop_fast = [&](auto active_c) __attribute__((always_inline)) {
    constexpr bool ACTIVE = decltype(active_c)::value;
    // offsets of the ring: the stage in use, the one after it, the one the next loads go to
    int boff = 0;
    for (int stage = 0; stage < ns; ++stage) {
      const int boff_next = boff == (NS - 1) * FSTAGE ? 0 : boff + FSTAGE;
      const int boff_fill = boff == 0 ? (NS - 1) * FSTAGE : boff - FSTAGE;  // stage + NS - 1
      const int step_next = boff_next - boff;
      static_for<R>([&](auto r_c) __attribute__((always_inline)) {
        constexpr int r = decltype(r_c)::value;
        constexpr bool last_r = r == R - 1;
        constexpr int rn = (r + 1) % R, rp = (r + R - 1) % R;
        constexpr int NPV = PS * DM;
        constexpr int NM = DS + NPV + (last_r ? NB : 0) + (MASKED ? 1 : 0);
        constexpr int NU = 8;
        // MFMA order: the P.V products of the last tile, (the bias products,) (the key mask,) the score products
        struct Order { int kind[NM], idx[NM]; };
        constexpr Order ord = [] {
          Order o{};
          int n = 0;
          for (int i = 0; i < NPV; ++i) { o.kind[n] = F_PV; o.idx[n++] = i; }
          if (last_r) for (int i = 0; i < NB; ++i) { o.kind[n] = F_B; o.idx[n++] = i; }
          if (MASKED) { o.kind[n] = F_M; o.idx[n++] = 0; }
          for (int i = 0; i < DS; ++i) { o.kind[n] = F_S; o.idx[n++] = i; }
          return o;
        }();
        if constexpr (ACTIVE) {
          SB();
          // operand reads: K rows of the next tile, V rows of this one, (the next stage's bias words)
          const uint32_t knext = last_r ? (uint32_t)step_next : (uint32_t)(rn * 32 * ROWB);
          frag kf[DS], vf[DM][PS], bwf[2];
#pragma unroll
          for (int sd = 0; sd < DS; ++sd) kf[sd] = lds_frag(ak[sd] + knext);
#pragma unroll
          for (int mt = 0; mt < DM; ++mt)
#pragma unroll
            for (int s2 = 0; s2 < PS; ++s2)
              vf[mt][s2] = lds_tr(avl[mt] + (uint32_t)(r * 32 * ROWB + 16 * s2 * ROWB), avh[mt] + (uint32_t)(r * 32 * ROWB + 16 * s2 * ROWB));
          if constexpr (last_r) {
            bwf[0] = lds_frag(ab + (uint32_t)step_next);
            bwf[1] = lds_frag(ab + (uint32_t)step_next + 1024u);
          }
          SB();
          f32x16 sc_next, bias_next = zero16();
          frag mk;
          if constexpr (MASKED) {
            // keys operand of the next tile's mask product (the next row of this stage, or the first row of the next)
            mk = kop.masked(last_r ? kwn[0] : kwc[rn]);
          }
          uint32_t pw[NU];
          const float mcr = mc[r], l_old = lrun[r];
          float l_new = l_old;  // the running row sum with this tile's probabilities on top
          // The arithmetic of a unit is a chain (fma -> exp2 -> conversion -> row sum), and a wave
          // that issues a dependent instruction right behind its producer waits for it: the
          // chain is cut into three steps that run one piece apart, so that between two MFMAs
          // the wave converts the units of the piece before, exponentiates its own and scales
          // those of the next.
          float xs[2 * NU], ps[2 * NU];
          auto scale_unit = [&](int u) __attribute__((always_inline)) {
            xs[2 * u] = __builtin_fmaf(sc_cur[2 * u], c, -mcr);
            xs[2 * u + 1] = __builtin_fmaf(sc_cur[2 * u + 1], c, -mcr);
          };
          auto exp_unit = [&](int u) __attribute__((always_inline)) {
            ps[2 * u] = fast_exp2(xs[2 * u]);
            ps[2 * u + 1] = fast_exp2(xs[2 * u + 1]);
          };
          auto pack_unit = [&](int u) __attribute__((always_inline)) {
            const pair_t w = {(T)ps[2 * u], (T)ps[2 * u + 1]};
            pw[u] = __builtin_bit_cast(uint32_t, w);
            l_new = pair_sum(w, ones, l_new);
          };
#pragma unroll
          for (int u = 0; u < NU / NM; ++u) scale_unit(u);
          SB();
          static_for<NM>([&](auto xc) __attribute__((always_inline)) {
            constexpr int x = decltype(xc)::value;
            constexpr int kind = ord.kind[x], idx = ord.idx[x];
            if constexpr (kind == F_B) {
              bias_next = E::mfma(bsel[idx / NPART][idx % NPART], bwf[idx / NPART], bias_next);
            } else if constexpr (kind == F_PV) {
              constexpr int s2 = idx / DM, mt = idx % DM;
              oacc[rp][mt] = E::mfma(vf_prev[mt][s2], pf_prev[s2], oacc[rp][mt]);
            } else if constexpr (kind == F_M) {
              sc_next = E::mfma(mk, qzero, last_r ? bias_next : bias_s);
            } else {
              if constexpr (idx == 0 && !MASKED) sc_next = E::mfma(kf[0], qf[rn][0], last_r ? bias_next : bias_s);
              else sc_next = E::mfma(kf[idx], qf[rn][idx], sc_next);
            }
            SB();
            if constexpr (x > 0) {
#pragma unroll
              for (int u = (x - 1) * NU / NM; u < x * NU / NM; ++u) pack_unit(u);
            }
#pragma unroll
            for (int u = x * NU / NM; u < (x + 1) * NU / NM; ++u) exp_unit(u);
            if constexpr (x + 1 < NM) {
#pragma unroll
              for (int u = (x + 1) * NU / NM; u < (x + 2) * NU / NM; ++u) scale_unit(u);
            } else {
#pragma unroll
              for (int u = x * NU / NM; u < (x + 1) * NU / NM; ++u) pack_unit(u);
            }
            SB();
          });
          if (__any(!(l_new - l_old <= kLazyLimit))) {
            // some query outgrew the reference: raise it to the running maximum and redo the tile
            // (the reference lives in the log2 domain only: mc = c * max)
            asm volatile("" ::);
            float mx = fmaxf(sc_cur[0], sc_cur[1]);
#pragma unroll
            for (int v = 2; v < 16; ++v) mx = fmaxf(mx, sc_cur[v]);
            mx = half_max(mx);
            // A row that attends to no key of this tile (the same for all its queries): every
            // score is the mask value alone.  The tile then adds nothing and must not become
            // the reference: exp2(c * score - reference) would be exp2 of the rounding error of
            // two numbers of the mask value's size.  (With a reference from real scores such a
            // tile's probabilities are exactly zero and it never gets here.)
            const bool no_key = MASKED && mx < 2.0f * E::kMaskElem;
            const float mcn = no_key ? mc[r] : fmaxf(mc[r], mx * c);
            const float alpha = fast_exp2(mc[r] - mcn);
#pragma unroll
            for (int mt = 0; mt < DM; ++mt)
#pragma unroll
              for (int v = 0; v < 16; ++v) oacc[r][mt][v] *= alpha;
            mc[r] = mcn;
            l_new = l_old * alpha;
#pragma unroll
            for (int u = 0; u < NU; ++u) {
              const float e0 = fast_exp2(__builtin_fmaf(sc_cur[2 * u], c, -mcn));
              const float e1 = fast_exp2(__builtin_fmaf(sc_cur[2 * u + 1], c, -mcn));
              const float p0 = no_key ? 0.f : e0, p1 = no_key ? 0.f : e1;
              const pair_t w = {(T)p0, (T)p1};
              pw[u] = __builtin_bit_cast(uint32_t, w);
              l_new = pair_sum(w, ones, l_new);
            }
          }
          lrun[r] = l_new;
#pragma unroll
          for (int s2 = 0; s2 < PS; ++s2) {
            pf_prev[s2] = __builtin_bit_cast(frag, (u32x4v){pw[4 * s2], pw[4 * s2 + 1], pw[4 * s2 + 2], pw[4 * s2 + 3]});
#pragma unroll
            for (int mt = 0; mt < DM; ++mt) vf_prev[mt][s2] = vf[mt][s2];
          }
          sc_cur = sc_next;
          if constexpr (last_r) bias_s = bias_next;
        }
        if constexpr (MASKED && last_r) {
#pragma unroll
          for (int r2 = 0; r2 < R; ++r2) kwc[r2] = kwn[r2];
          fetch_keep_words(stage + 2, kwn);
        }
        // The next slot reads stage s+1: every wave's loads of it have landed (a ring of four
        // leaves one younger stage in flight), and nobody reads stage s-1 any more: the buffer
        // that the loads issued in the next slot overwrite.
        if constexpr (r == R - 2) ring_sync<(NS - 3) * NLD>();
        if constexpr (last_r) issue_fast(boff_fill);
      });
      // the ring moves on
#pragma unroll
      for (int sd = 0; sd < DS; ++sd) ak[sd] += (uint32_t)step_next;
#pragma unroll
      for (int mt = 0; mt < DM; ++mt) {
        avl[mt] += (uint32_t)step_next;
        avh[mt] += (uint32_t)step_next;
      }
      ab += (uint32_t)step_next;
      boff = boff_next;
    }
    };
    if (wave_active) stage_loop_fast(std::true_type{});
    else stage_loop_fast(std::false_type{});
    // P.V of the last tile
    if (wave_active) {
#pragma unroll
      for (int s2 = 0; s2 < PS; ++s2)
#pragma unroll
        for (int mt = 0; mt < DM; ++mt) oacc[R - 1][mt] = E::mfma(vf_prev[mt][s2], pf_prev[s2], oacc[R - 1][mt]);
    }
    wait_dma();  // (the last prefetches are still on their way into LDS)
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
  bool fast = false, fast_masked = false;
  if constexpr (FAST) {
    // (the per-lane offsets of the stage loads are 32-bit: rows and keys of a stage must lie within 4 GiB)
    const auto fits = [&](const Str5& st) {
      return st.i >= 0 && st.j >= 0 && (uint64_t)(R - 1) * st.i + 31ull * st.j + D < (1ull << 31) / sizeof(T);
    };
    const bool shape_fits = (N & 31) == 0 && fits(a.sk) && fits(a.sv);
    fast = shape_fits && masks.all_plain();
    // (a fully masked row drops its bias and q.k: such workgroups take the general loop)
    fast_masked = shape_fits && !fast && !any_flagged && masks.last_live() > 0;
  }
  if (fast) {
    if constexpr (FAST) fast_loop(std::false_type{});
  } else if (fast_masked) {
    if constexpr (FAST) fast_loop(std::true_type{});
  } else {
    setup_general();
    if (masks.all_plain() && ntiles % KU == 0) stage_loop(std::integral_constant<int, kPlain>{});
    else if (!any_flagged) stage_loop(std::integral_constant<int, kMasked>{});
    else stage_loop(std::integral_constant<int, kGeneral>{});
  }

  if (!wave_active) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = i0 + r;
    const float ltot = half_sum(lrun[r]);
    if (i >= N) continue;  // (wave-uniform; the lanes of queries past the end stay for the exchange inside the store)
    T* orow = reinterpret_cast<T*>(a.o) + (((int64_t)bh * N + i) * N) * D;
    store_rows_any<T, D, DM>(orow + (int64_t)j * D, oacc[r], 1.0f / ltot, g, j < N);
    if (g == 0 && j < N) {
      float lse = kLn2 * (mc[r] + fast_log2(ltot));
      if (flagged[r]) lse = a.neg_inf + lse;
      a.lse[((int64_t)bh * N + i) * N + j] = lse;
    }
  }
}

}  // namespace tri
