// Backward kernel 3 of 3: db[j, k] = sum over rows i of dS[i, j, k].
//
// Work unit: (batch*head, block of 2*WJ*32 queries j, block of 2*WK*32 keys k,
// chunk of pair rows i).  The 2 x 2 waves of a workgroup each own WJ x WK tiles of
// 32 x 32 and keep their db tiles in fp32 registers while the workgroup walks its
// rows, so the reduction over i has one fixed order and needs no atomics.  The
// bias tiles (register-resident, fp32, raw-score domain) are the accumulator init
// of the score MFMA of every row.  Per row the workgroup stages the Q, dO rows of
// its queries and the K, V rows of its keys in LDS (direct global->LDS loads,
// double-buffered, swizzled), and each wave recomputes for its tiles
//   S^T = K Q^T (+bias), P^T = exp2(S^T c - lse), dP^T = V dO^T, dS^T = P^T (dP^T - delta)
// with every operand in its natural row-major layout, adding dS^T into db.
// When the rows are split into several chunks (to fill the GPU at small n), each
// chunk writes an fp32 partial and a second kernel adds the partials in order.
//
// Replaces _bwd_b of reference src/trifast/triton.py:394-501.
#pragma once
#include "tri_args.hpp"
#include "tri_common.hpp"
#include "tri_tile.hpp"

namespace tri {

template <typename T, int D, int WJ, int WK, int NBUF>
__global__ __launch_bounds__(256) void tri_bwd_b_kernel(const BwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using Tile = LdsTile<T, D>;
  constexpr int KP = E::KP;
  constexpr int DS = D / (2 * KP);
  constexpr int NW = 4;
  constexpr int BJ = 2 * WJ * 32, BKB = 2 * WK * 32;  // queries / keys per workgroup
  constexpr int ROWB = Tile::ROWB;
  // one stage: Q rows | dO rows | K rows | V rows | lse[BJ] | delta[BJ] | row meta
  // (64 words: the WKW keep words of the key block, then the row's flag)
  constexpr int OFF_Q = 0, OFF_DO = BJ * ROWB, OFF_K = 2 * BJ * ROWB, OFF_V = OFF_K + BKB * ROWB;
  constexpr int OFF_LSE = OFF_V + BKB * ROWB, OFF_DELTA = OFF_LSE + BJ * 4;
  constexpr int OFF_META = OFF_DELTA + BJ * 4;
  constexpr int STAGE = OFF_META + 256;
  constexpr int WKW = BKB / 32;

  extern __shared__ __attribute__((aligned(16))) unsigned char tri_smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int jl = lane & 31, g = lane >> 5;
  const int N = a.N;
  const int bh = blockIdx.z % a.BH, chunk = blockIdx.z / a.BH;
  const int b = bh / a.H, h = bh % a.H;
  const int j_blk = blockIdx.x * BJ, k_blk = blockIdx.y * BKB;
  const int wj = wave & 1, wk = wave >> 1;
  const int j_wave = j_blk + wj * (WJ * 32), k_wave = k_blk + wk * (WK * 32);
  const int i_begin = chunk * a.rows_per_chunk;
  const int i_end = min(N, i_begin + a.rows_per_chunk);
  const int nrows = i_end - i_begin;

  const T* qbase = reinterpret_cast<const T*>(a.q) + b * a.sq.b + h * a.sq.h;
  const T* kbase = reinterpret_cast<const T*>(a.k) + b * a.sk.b + h * a.sk.h;
  const T* vbase = reinterpret_cast<const T*>(a.v) + b * a.sv.b + h * a.sv.h;
  const T* dobase = reinterpret_cast<const T*>(a.dout) + b * a.sdo.b + h * a.sdo.h;
  const T* pack_bh = reinterpret_cast<const T*>(a.packq) + (int64_t)bh * a.NP * a.NP * 1024;
  const float* lse_bh = a.lse + (int64_t)bh * N * N;
  const float* delta_bh = a.delta + (int64_t)bh * N * N;

  // bias tiles in the raw-score domain: accumulator init of every row's score MFMA
  f32x16 biasr[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk)
      biasr[tj][tk] = bias_tile<T>(pack_bh, a.NP, min((j_wave >> 5) + tj, a.NP - 1), min((k_wave >> 5) + tk, a.NP - 1), lane, a.sqrt_d, 0.f);

  f32x16 dbacc[WJ][WK];
#pragma unroll
  for (int tj = 0; tj < WJ; ++tj)
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) dbacc[tj][tk] = zero16();

  // issue the loads of row i into stage buffer `buf` (indices clamped, never branched)
  auto issue_row = [&](int i, int buf) {
    unsigned char* st = tri_smem + buf * STAGE;
    i = min(i, N - 1);
    Tile::template fill<BJ, NW>(st + OFF_Q, [&](int r) { return qbase + i * a.sq.i + (int64_t)min(j_blk + r, N - 1) * a.sq.j; }, wave, lane);
    Tile::template fill<BJ, NW>(st + OFF_DO, [&](int r) { return dobase + i * a.sdo.i + (int64_t)min(j_blk + r, N - 1) * a.sdo.j; }, wave, lane);
    Tile::template fill<BKB, NW>(st + OFF_K, [&](int r) { return kbase + i * a.sk.i + (int64_t)min(k_blk + r, N - 1) * a.sk.j; }, wave, lane);
    Tile::template fill<BKB, NW>(st + OFF_V, [&](int r) { return vbase + i * a.sv.i + (int64_t)min(k_blk + r, N - 1) * a.sv.j; }, wave, lane);
    fill_floats<BJ, NW>(reinterpret_cast<float*>(st + OFF_LSE), [&](int x) { return lse_bh + (int64_t)i * N + min(j_blk + x, N - 1); }, wave, lane);
    fill_floats<BJ, NW>(reinterpret_cast<float*>(st + OFF_DELTA), [&](int x) { return delta_bh + (int64_t)i * N + min(j_blk + x, N - 1); }, wave, lane);
    if (wave == NW - 1) {
      // lanes 0..WKW-1: keep words of this key block; lane WKW: the row flag
      const uint32_t* src = (lane == WKW) ? a.rowflag + (int64_t)b * N + i
                                          : a.keep + ((int64_t)b * N + i) * a.nwords + min(k_blk / 32 + min(lane, WKW - 1), a.nwords - 1);
      __builtin_amdgcn_global_load_lds((const TRI_G1 void*)src, (TRI_L3 void*)(st + OFF_META), 4, 0, 0);
    }
  };

  const float c = a.c;
  const float lse2_flagged = fast_log2((float)N);
  const bool wave_live = j_wave < N && k_wave < N;

  auto compute_row = [&](int buf) {
    const unsigned char* st = tri_smem + buf * STAGE;
    const uint32_t* meta = reinterpret_cast<const uint32_t*>(st + OFF_META);
    const bool flagged = meta[WKW] != 0;
    // operands of this wave's tiles; tile row m of the key tiles stands for key perm32(m)
    frag qf[WJ][DS], dof[WJ][DS], kf[WK][DS], vf[WK][DS];
    float lse2[WJ], delta[WJ];
#pragma unroll
    for (int tj = 0; tj < WJ; ++tj) {
      const int r = wj * (WJ * 32) + 32 * tj + jl;
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        // a fully masked row ignores q.k as well as the bias
        qf[tj][s] = flagged ? E::zero() : Tile::operand(st + OFF_Q, r, s, g);
        dof[tj][s] = Tile::operand(st + OFF_DO, r, s, g);
      }
      lse2[tj] = flagged ? lse2_flagged : reinterpret_cast<const float*>(st + OFF_LSE)[r] * kLog2e;
      delta[tj] = reinterpret_cast<const float*>(st + OFF_DELTA)[r];
    }
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
      const int r = wk * (WK * 32) + 32 * tk + perm32(jl);
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        kf[tk][s] = Tile::operand(st + OFF_K, r, s, g);
        vf[tk][s] = Tile::operand(st + OFF_V, r, s, g);
      }
    }
#pragma unroll
    for (int tk = 0; tk < WK; ++tk) {
      // a key tile past the last word of the row has no attended key
      const uint32_t keepw = (k_wave / 32 + tk < a.nwords) ? meta[wk * WK + tk] : 0u;
      if (keepw == 0) continue;  // no attended key in this tile: dS = 0
      const bool mixed = keepw != 0xffffffffu;
#pragma unroll
      for (int tj = 0; tj < WJ; ++tj) {
        f32x16 s;
        if (mixed) {
          s = mask_tile(keepw, g);
          if (!flagged) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s[v] += biasr[tj][tk][v];
          }
          s = E::mfma(kf[tk][0], qf[tj][0], s);
        } else if (flagged) {
          s = E::mfma(kf[tk][0], qf[tj][0], zero16());
        } else {
          s = E::mfma(kf[tk][0], qf[tj][0], biasr[tj][tk]);
        }
        f32x16 dp = E::mfma(vf[tk][0], dof[tj][0], zero16());
#pragma unroll
        for (int sd = 1; sd < DS; ++sd) {
          s = E::mfma(kf[tk][sd], qf[tj][sd], s);
          dp = E::mfma(vf[tk][sd], dof[tj][sd], dp);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = fast_exp2(__builtin_fmaf(s[v], c, -lse2[tj]));
          dbacc[tj][tk][v] = __builtin_fmaf(p, dp[v] + delta[tj], dbacc[tj][tk][v]);  // the workspace holds -delta
        }
      }
    }
  };

  if constexpr (NBUF == 2) {
    issue_row(i_begin, 0);
    wait_dma();
    __syncthreads();
    for (int ir = 0; ir < nrows; ir += 2) {
      issue_row(i_begin + ir + 1, 1);
      if (wave_live) compute_row(0);
      wait_dma();
      __syncthreads();
      if (ir + 1 >= nrows) break;
      issue_row(i_begin + ir + 2, 0);
      if (wave_live) compute_row(1);
      wait_dma();
      __syncthreads();
    }
  } else {
    // one stage only (the double buffer does not fit in LDS): load, then compute
    for (int ir = 0; ir < nrows; ++ir) {
      issue_row(i_begin + ir, 0);
      wait_dma();
      __syncthreads();
      if (wave_live) compute_row(0);
      __syncthreads();
    }
  }
  if (!wave_live) return;

  // a single chunk writes db itself; several chunks write fp32 partials
  const bool direct = a.nchunks == 1;
  T* db_bh = reinterpret_cast<T*>(a.db) + (int64_t)bh * N * N;
  float* part = a.dbpart + ((int64_t)chunk * a.BH + bh) * N * N;
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
        if (!direct) {
          float* dst = part + (int64_t)j * N + key0;
          if (vec_store && key0 + 8 <= N) {
#pragma unroll
            for (int e4 = 0; e4 < 2; ++e4) {
              f32x4 ov;
#pragma unroll
              for (int e = 0; e < 4; ++e) ov[e] = dbacc[tj][tk][8 * r + 4 * e4 + e];
              *reinterpret_cast<f32x4*>(dst + 4 * e4) = ov;
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (key0 + e < N) dst[e] = dbacc[tj][tk][8 * r + e];
          }
          continue;
        }
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

// db = sum over chunks of the fp32 partials, in chunk order
template <typename T>
__global__ __launch_bounds__(256) void tri_bwd_b_reduce_kernel(const float* part, T* db, int64_t count, int nchunks) {
  const int64_t x = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (x >= count) return;
  float acc = part[x];
  for (int ch = 1; ch < nchunks; ++ch) acc += part[(int64_t)ch * count + x];
  db[x] = (T)acc;
}

}  // namespace tri
