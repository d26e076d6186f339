// Weight gradient of a linear layer over a pair representation,
//   dW[n, k] = sum over r of dY[r, n] * x[r, k]        x [rows, K], dY [rows, N], dW [N, K]
// for the tall, narrow shapes a triangle-attention block has: rows = b n^2 in the millions,
// K and N a few hundred at most.  The contraction runs over the long dimension and the
// result is tiny, which is the one shape of the block's six linear layers that a BLAS library
// serves badly (one or two workgroups walk all the rows: 1.7 ms per layer at rows = 2^20,
// K = N = 128, against 0.15 ms for the layer's other two products).  Here the rows are
// split into chunks, one workgroup per (chunk, group of 128 output rows n): it streams its
// rows of dY and x through LDS 32 at a time (both operands have the contraction index as
// their memory row, so both are read back transposed, ds_read_tr), keeps its part of dW in
// fp32 accumulators (wave w: rows n of its 32-block, all K columns), and writes it as an fp32
// partial; a second kernel adds the partials in a fixed order (deterministic, no atomics)
// and rounds once.  The layer's bias gradient, the column sums of dY, comes out of the same
// pass on request (dY^T times a vector of ones: one more MFMA per 16 rows).  Bound by HBM: every element of dY and x is read once per group of n.
// No counterpart in the reference: the linear layers around its operator are only hinted
// at by the module of reference tests/unit/test_trifast.py:152-169.
#pragma once
#include <type_traits>

#include "tri_common.hpp"
#include "tri_dispatch.hpp"

namespace tri {

// A layer's output (or output gradient) is [rows, N] or, "heads outermost", [N / hd][rows][hd]:
// the layout the attention operator reads q, k, v in (and writes dq, dk, dv in) without the
// two heads of a 128-byte line belonging to different workgroups.  hd = 0: plain.
// (hd is a multiple of 8 and divides N, so a 16-byte piece never straddles two heads.)
TRI_DEV int64_t linear_offset(int64_t row, int col, int N, int hd, int64_t rows) {
  return hd ? ((int64_t)(col / hd) * rows + row) * hd + col % hd : row * N + col;
}

struct LinearDwArgs {
  const void* x;    // [rows, K]
  const void* dy;   // [rows, N] (see linear_offset)
  int hd;
  float* part;      // [chunks, N, K] partial sums
  void* dw;         // [N, K]
  float* part_b;    // [chunks, N] partial column sums of dy (the layer's bias gradient), or null
  void* db;         // [N], or null
  int64_t rows;
  int64_t rows_per_chunk;  // multiple of 32
  int chunks;
  int K, N;
};

constexpr int kLinearRowsPerStep = 32;

// rows of one chunk: at least 1024 (the partials of a chunk cost as much traffic as 128 rows),
// and at most 768 chunks: three workgroups per CU are resident at once, and a grid that is not
// a whole number of such rounds leaves CUs idle in the last one
inline int64_t linear_dw_rows_per_chunk(int64_t rows) {
  const int64_t per = ((rows + 767) / 768 + 31) / 32 * 32;
  return per < 1024 ? 1024 : per;
}
inline int64_t linear_dw_chunks(int64_t rows) {
  const int64_t per = linear_dw_rows_per_chunk(rows);
  return (rows + per - 1) / per;
}

// KD: columns of x (K, one of 32, 64, 128, 256); ND: output rows n per workgroup, 128 (wave w
// owns rows 32 w .. 32 w + 31 and every column block of x) or, for layers of up to 32 outputs,
// 32 (the four waves share the column blocks of x)
template <typename T, int KD, int ND, bool BIAS>
__global__ __launch_bounds__(256) void linear_dw_kernel(const LinearDwArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using vec = typename E::vec;
  constexpr int KB = KD / 32;            // 32-column blocks of x
  constexpr bool SPLIT_K = ND == 32;
  constexpr int KBW = SPLIT_K ? (KB + 3) / 4 : KB;  // column blocks of one wave
  constexpr int LDX = KD + 8, LDY = ND + 8;  // padded rows (16-byte multiples)
  constexpr int XCH = 32 * KD / 8, YCH = 32 * ND / 8;          // 16-byte chunks of a step's tiles
  constexpr int XC = (XCH + 255) / 256, YC = (YCH + 255) / 256;  // ... per lane
  __shared__ __attribute__((aligned(16))) T xs[2][32][LDX];
  __shared__ __attribute__((aligned(16))) T ys[2][32][LDY];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int K = KD, N = a.N;
  const int n_grp = blockIdx.y * ND;  // first output row of this workgroup
  const int64_t r_begin = (int64_t)blockIdx.x * a.rows_per_chunk;
  const int64_t r_end = min(a.rows, r_begin + a.rows_per_chunk);
  const int steps = (int)((r_end - r_begin + 31) / 32);
  const T* xg = reinterpret_cast<const T*>(a.x);
  const T* yg = reinterpret_cast<const T*>(a.dy);
  const bool y_vec = (N % 8) == 0;  // rows of dY keep 16-byte alignment

  // this lane's chunks of a step's tiles (tile row, first column), fetched two steps ahead of
  // their use: one set of registers per step in flight
  vec xr2[2][XC], yr2[2][YC];
  auto load_step = [&](int s, vec* xr, vec* yr) {
    const int64_t r0 = r_begin + 32 * (int64_t)s;
#pragma unroll
    for (int c = 0; c < XC; ++c) {
      const int p = c * 256 + tid, r = p / (KD / 8), col = 8 * (p % (KD / 8));
      vec v = {};
      if (p < XCH && r0 + r < r_end) v = *reinterpret_cast<const vec*>(xg + (r0 + r) * K + col);
      xr[c] = v;
    }
#pragma unroll
    for (int c = 0; c < YC; ++c) {
      const int p = c * 256 + tid, r = p / (ND / 8), col = n_grp + 8 * (p % (ND / 8));
      vec v = {};
      if (p < YCH && r0 + r < r_end && col < N) {
        const T* src = yg + linear_offset(r0 + r, col, N, a.hd, a.rows);
        if (y_vec) {
          v = *reinterpret_cast<const vec*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N) v[e] = src[e];
        }
      }
      yr[c] = v;
    }
  };
  auto store_step = [&](int buf, const vec* xr, const vec* yr) {
#pragma unroll
    for (int c = 0; c < XC; ++c) {
      const int p = c * 256 + tid, r = p / (KD / 8), col = 8 * (p % (KD / 8));
      if (p < XCH) *reinterpret_cast<vec*>(&xs[buf][r][col]) = xr[c];
    }
#pragma unroll
    for (int c = 0; c < YC; ++c) {
      const int p = c * 256 + tid, r = p / (ND / 8), col = 8 * (p % (ND / 8));
      if (p < YCH) *reinterpret_cast<vec*>(&ys[buf][r][col]) = yr[c];
    }
  };

  f32x16 acc[KBW];
#pragma unroll
  for (int i = 0; i < KBW; ++i) acc[i] = zero16();
  const int n_blk = SPLIT_K ? 0 : wave;                          // this wave's 32 output rows
  auto col_block = [&](int i) { return SPLIT_K ? wave + 4 * i : i; };  // ... and its column blocks of x
  // (a wave whose output rows lie past N, or that has no column block, only stages)
  const bool wave_live = __builtin_amdgcn_readfirstlane((int)(n_grp + 32 * n_blk < N && col_block(0) < KB)) != 0;
  // the bias gradient, the column sums of dy, rides along as one more product: dy^T times ones
  // (one wave per 32 output rows does it)
  const bool sums = BIAS && (!SPLIT_K || wave == 0);
  const frag ones = E::splat(1.0f);
  f32x16 bacc = zero16();

  load_step(0, xr2[0], yr2[0]);
  if (steps > 1) load_step(1, xr2[1], yr2[1]);
  store_step(0, xr2[0], yr2[0]);
  __syncthreads();
  auto one_step = [&](int s, auto parity) __attribute__((always_inline)) {
    constexpr int buf = decltype(parity)::value;  // s % 2: the LDS buffer of step s, the register set of step s + 2
    if (s + 2 < steps) load_step(s + 2, xr2[buf], yr2[buf]);
    if (wave_live) {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        // A: dY^T (output row n in the lane, 8 memory rows as contraction slots); B: x^T
        const frag af = lds_tr_frag<T, LDY>(ys[buf], 16 * s2 + 8 * g, 32 * n_blk, lane);
        if (sums) bacc = E::mfma(af, ones, bacc);
#pragma unroll
        for (int i = 0; i < KBW; ++i) {
          if (col_block(i) < KB) {
            const frag bf = lds_tr_frag<T, LDX>(xs[buf], 16 * s2 + 8 * g, 32 * col_block(i), lane);
            acc[i] = E::mfma(af, bf, acc[i]);
          }
        }
      }
    }
    // the other buffer was last read in step s - 1, which every wave left before the
    // barrier that ended it
    if (s + 1 < steps) store_step(buf ^ 1, xr2[buf ^ 1], yr2[buf ^ 1]);
    __syncthreads();
  };
  for (int s = 0; s < steps; s += 2) {
    one_step(s, std::integral_constant<int, 0>{});
    if (s + 1 < steps) one_step(s + 1, std::integral_constant<int, 1>{});
  }
  if (!wave_live) return;
  // partial [chunk][n][k]: the lane holds column k = 32 kb + lane % 32 and rows
  // n = 32 wave + 8 q + 4 g + e of the group
  if (sums && (lane & 31) == 0) {
    // (every column of the product holds the same sums: lanes 0 and 32 store theirs)
    float* pb = a.part_b + (int64_t)blockIdx.x * N;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int n = n_grp + 32 * n_blk + 8 * (v / 4) + 4 * g + (v % 4);
      if (n < N) pb[n] = bacc[v];
    }
  }
  float* part = a.part + (int64_t)blockIdx.x * N * K;
#pragma unroll
  for (int i = 0; i < KBW; ++i) {
    if (col_block(i) >= KB) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int n = n_grp + 32 * n_blk + 8 * (v / 4) + 4 * g + (v % 4);
      if (n < N) part[(int64_t)n * K + 32 * col_block(i) + (lane & 31)] = acc[i][v];
    }
  }
}

// dW = sum of the partials, rounded once.  A workgroup sums 32 elements: lane group c of 8
// adds the chunks c, c + 8, ... in increasing order, then the 8 sums are added in order of c
// (one fixed association, whatever the timing).
template <typename T>
__global__ __launch_bounds__(256) void linear_dw_reduce_kernel(const float* part, T* out, int64_t count, int chunks) {
  __shared__ float sums[8][32];
  const int e = threadIdx.x & 31, c0 = threadIdx.x >> 5;
  const int64_t idx = (int64_t)blockIdx.x * 32 + e;
  float sum = 0.f;
  if (idx < count) {
#pragma unroll 4
    for (int c = c0; c < chunks; c += 8) sum += part[(int64_t)c * count + idx];
  }
  sums[c0][e] = sum;
  __syncthreads();
  if (c0 == 0 && idx < count) {
    float total = sums[0][e];
#pragma unroll
    for (int c = 1; c < 8; ++c) total += sums[c][e];
    out[idx] = (T)total;
  }
}

inline bool linear_dw_k_ok(int64_t k) { return k == 32 || k == 64 || k == 128 || k == 256; }

template <typename T>
inline hipError_t linear_dw_launch_t(const LinearDwArgs& a, hipStream_t st) {
  const dim3 block(256);
  const bool split_k = a.N <= 32;
  const dim3 grid((unsigned)a.chunks, split_k ? 1u : (unsigned)((a.N + 127) / 128));
#define TRI_DW_CASE(KD)                                                                                          \
  case KD:                                                                                                       \
    if (split_k && a.part_b) hipLaunchKernelGGL((linear_dw_kernel<T, KD, 32, true>), grid, block, 0, st, a);     \
    else if (split_k) hipLaunchKernelGGL((linear_dw_kernel<T, KD, 32, false>), grid, block, 0, st, a);           \
    else if (a.part_b) hipLaunchKernelGGL((linear_dw_kernel<T, KD, 128, true>), grid, block, 0, st, a);          \
    else hipLaunchKernelGGL((linear_dw_kernel<T, KD, 128, false>), grid, block, 0, st, a);                       \
    break;
  switch (a.K) {
    TRI_DW_CASE(32)
    TRI_DW_CASE(64)
    TRI_DW_CASE(128)
    TRI_DW_CASE(256)
    default: return hipErrorInvalidConfiguration;
  }
#undef TRI_DW_CASE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int64_t count = (int64_t)a.N * a.K;
  hipLaunchKernelGGL((linear_dw_reduce_kernel<T>), dim3((unsigned)((count + 31) / 32)), block, 0, st, (const float*)a.part, reinterpret_cast<T*>(a.dw), count, a.chunks);
  e = hipGetLastError();
  if (e != hipSuccess || !a.part_b) return e;
  hipLaunchKernelGGL((linear_dw_reduce_kernel<T>), dim3((unsigned)((a.N + 31) / 32)), block, 0, st, (const float*)a.part_b, reinterpret_cast<T*>(a.db), (int64_t)a.N, a.chunks);
  return hipGetLastError();
}

inline hipError_t linear_dw_launch(const LinearDwArgs& a, int dtype, hipStream_t st) {
  switch (dtype) {
    case kBF16: return linear_dw_launch_t<__bf16>(a, st);
    case kF16: return linear_dw_launch_t<_Float16>(a, st);
  }
  return hipErrorInvalidConfiguration;
}

}  // namespace tri

namespace tri {

// ---------------------------------------------------------------------------------------
// Input gradient of several linear layers over one input,
//   dx[r, :] = sum over layers p of dy_p[r, :] W_p            dy_p [rows, N_p], W_p [N_p, K]
// in one pass: every dy_p is read once and dx is written once (the BLAS library runs one
// product per layer and autograd adds them up, which moves dx through memory nine times
// for five layers).  A workgroup owns 256 rows (wave w: rows 64 w .. 64 w + 63 as two 32-row
// tiles) and all K columns, accumulated in fp32 registers over the layers; the dy rows are
// staged through LDS 32 columns at a time (coalesced 16-byte loads, two stages ahead in
// registers), and so are the same 32 columns of the weights, which come as W_p^T [K, N_p]
// (made once per call by the caller: a few tens of KiB) so that the operand fragments of both
// are plain 16-byte LDS reads.  (Weight fragments loaded straight from global memory, eight
// per chunk and wave, were waited for one by one: 0.59 ms for the block's five layers.)  The product is computed transposed (W^T dy^T): a lane ends up with one row of dx
// and 4 x 4 consecutive columns per column block, stored as 8-byte pieces.
// ---------------------------------------------------------------------------------------
constexpr int kLinearLayers = 6;

struct LinearDxArgs {
  const void* dy[kLinearLayers];   // [rows, n[p]] (see linear_offset)
  const void* wt[kLinearLayers];   // [K, n[p]]: W_p transposed
  int n[kLinearLayers];
  int hd[kLinearLayers];
  int nlayers;
  void* dx;                        // [rows, K]
  int64_t rows;
  int K;
};

template <typename T, int KD>
__global__ __launch_bounds__(256) void linear_dx_kernel(const LinearDxArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using vec = typename E::vec;
  constexpr int KB = KD / 32;       // 32-column blocks of dx
  constexpr int RT = 2;             // 32-row tiles per wave
  constexpr int ROWS = 4 * RT * 32;  // rows per workgroup
  constexpr int LD = 32 + 8;        // padded row of a staged chunk (32 columns of dy)
  constexpr int CH = ROWS * 32 / 8 / 256;  // 16-byte pieces of a chunk per lane
  constexpr int PF = 2;             // chunks in flight: one register set and one LDS buffer each
  constexpr int WPC = KD * 32 / 8;  // 16-byte pieces of a chunk of W^T (KD rows of 32 columns)
  constexpr int WCH = (WPC + 255) / 256;
  __shared__ __attribute__((aligned(16))) T ys[PF][ROWS][LD];
  __shared__ __attribute__((aligned(16))) T ws[PF][KD][LD];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cl = lane & 31, g = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;

  // the chunks of all layers, in order: chunk c of layer p covers its columns 32 c .. 32 c + 31
  int total = 0;
  for (int p = 0; p < a.nlayers; ++p) total += (a.n[p] + 31) / 32;

  vec yr[PF][CH], wr[PF][WCH];
  // (layer, first column) of chunk number q, walked incrementally by the two users below
  struct Cursor {
    int p, c;
  };
  auto advance = [&](Cursor& cur) {
    if (32 * (cur.c + 1) < a.n[cur.p]) ++cur.c;
    else { ++cur.p; cur.c = 0; }
  };
  auto load_chunk = [&](const Cursor& cur, vec* dst, vec* wdst) {
    const T* src = reinterpret_cast<const T*>(a.dy[cur.p]);
    const T* wsrc = reinterpret_cast<const T*>(a.wt[cur.p]);
    const int N = a.n[cur.p];
    const bool vec_ok = (N % 8) == 0;
    // the same 32 columns of W^T (columns past N_p are zero, like those of dy)
#pragma unroll
    for (int x = 0; x < WCH; ++x) {
      const int q = x * 256 + tid, k = q / 4, col = 32 * cur.c + 8 * (q % 4);
      vec v = {};
      if (q < WPC && col < N) {
        const T* s = wsrc + (int64_t)k * N + col;
        if (vec_ok) {
          v = *reinterpret_cast<const vec*>(s);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N) v[e] = s[e];
        }
      }
      wdst[x] = v;
    }
#pragma unroll
    for (int x = 0; x < CH; ++x) {
      const int q = x * 256 + tid, r = q / 4, col = 32 * cur.c + 8 * (q % 4);
      vec v = {};
      if (row0 + r < a.rows && col < N) {
        const T* s = src + linear_offset(row0 + r, col, N, a.hd[cur.p], a.rows);
        if (vec_ok) {
          v = *reinterpret_cast<const vec*>(s);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (col + e < N) v[e] = s[e];
        }
      }
      dst[x] = v;
    }
  };
  auto store_chunk = [&](int buf, const vec* src, const vec* wsrc) {
#pragma unroll
    for (int x = 0; x < CH; ++x) {
      const int q = x * 256 + tid, r = q / 4, col = 8 * (q % 4);
      *reinterpret_cast<vec*>(&ys[buf][r][col]) = src[x];
    }
#pragma unroll
    for (int x = 0; x < WCH; ++x) {
      const int q = x * 256 + tid, k = q / 4, col = 8 * (q % 4);
      if (q < WPC) *reinterpret_cast<vec*>(&ws[buf][k][col]) = wsrc[x];
    }
  };

  f32x16 acc[RT][KB];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) acc[t][kb] = zero16();

  Cursor ld{0, 0};
#pragma unroll
  for (int q = 0; q < PF; ++q)
    if (q < total) { load_chunk(ld, yr[q], wr[q]); advance(ld); }
  store_chunk(0, yr[0], wr[0]);
  __syncthreads();
  // chunk q: registers and LDS buffer q % PF.  Its registers went to LDS at the end of the
  // step before, so they take the loads of chunk q + PF; the buffer of chunk q + 1 was last
  // read in step q + 1 - PF, which every wave left at least one barrier ago.
  auto one_chunk = [&](int q, auto which) __attribute__((always_inline)) {
    constexpr int buf = decltype(which)::value;
    constexpr int nxt = (buf + 1) % PF;
    if (q + PF < total) { load_chunk(ld, yr[buf], wr[buf]); advance(ld); }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      frag bf[RT];
#pragma unroll
      for (int t = 0; t < RT; ++t) bf[t] = *reinterpret_cast<const frag*>(&ys[buf][64 * wave + 32 * t + cl][16 * s2 + 8 * g]);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        // W^T[k][32 c + 16 s2 + 8 g ..], k = 32 kb + lane % 32
        const frag af = *reinterpret_cast<const frag*>(&ws[buf][32 * kb + cl][16 * s2 + 8 * g]);
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[t][kb] = E::mfma(af, bf[t], acc[t][kb]);
      }
    }
    if (q + 1 < total) store_chunk(nxt, yr[nxt], wr[nxt]);
    __syncthreads();
  };
  for (int q = 0; q < total; q += PF) {
    one_chunk(q, std::integral_constant<int, 0>{});
    if (q + 1 < total) one_chunk(q + 1, std::integral_constant<int, 1>{});
  }

  // dx: the lane holds row 64 wave + 32 t + lane % 32 and columns 32 kb + 8 q + 4 g + 0..3
  T* dx = reinterpret_cast<T*>(a.dx);
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int64_t row = row0 + 64 * wave + 32 * t + cl;
    if (row >= a.rows) continue;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        typename E::vec4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (T)acc[t][kb][4 * q + e];
        *reinterpret_cast<typename E::vec4*>(dx + row * KD + 32 * kb + 8 * q + 4 * g) = ov;
      }
  }
}

template <typename T>
inline hipError_t linear_dx_launch_t(const LinearDxArgs& a, hipStream_t st) {
  const dim3 grid((unsigned)((a.rows + 255) / 256)), block(256);
  switch (a.K) {
    case 32: hipLaunchKernelGGL((linear_dx_kernel<T, 32>), grid, block, 0, st, a); break;
    case 64: hipLaunchKernelGGL((linear_dx_kernel<T, 64>), grid, block, 0, st, a); break;
    case 128: hipLaunchKernelGGL((linear_dx_kernel<T, 128>), grid, block, 0, st, a); break;
    default: return hipErrorInvalidConfiguration;
  }
  return hipGetLastError();
}

// (the accumulators of 64 rows x K columns per wave stay in registers: K up to 128)
inline bool linear_dx_k_ok(int64_t k) { return k == 32 || k == 64 || k == 128; }

inline hipError_t linear_dx_launch(const LinearDxArgs& a, int dtype, hipStream_t st) {
  switch (dtype) {
    case kBF16: return linear_dx_launch_t<__bf16>(a, st);
    case kF16: return linear_dx_launch_t<_Float16>(a, st);
  }
  return hipErrorInvalidConfiguration;
}

}  // namespace tri

namespace tri {

// ---------------------------------------------------------------------------------------
// Several linear layers over one input in one pass,
//   y_p[r, :] = x[r, :] W_p^T + bias_p        x [rows, K], W_p [N_p, K], y_p [rows, N_p]
// x is read once for all layers (the BLAS library reads it once per layer).  A workgroup
// owns 256 rows: their K / 16 operand fragments go through LDS once (coalesced loads) into
// registers (wave w: rows 64 w .. 64 w + 63 as two 32-row tiles) and stay there; the layers'
// weights pass through LDS 128 output columns at a time (the next group ahead in registers).  The
// product is computed transposed (W x^T, bias as accumulator init), so a lane holds one row
// and 4 x 4 consecutive columns of the chunk; the chunk goes back through the wave's own
// piece of LDS and leaves as 16-byte pieces, 64 contiguous bytes per row.
// ---------------------------------------------------------------------------------------
struct LinearFwdArgs {
  const void* x;                    // [rows, K]
  const void* w[kLinearLayers];     // [n[p], K]
  const void* bias[kLinearLayers];  // [n[p]] or null
  void* y[kLinearLayers];           // [rows, n[p]] (see linear_offset)
  int n[kLinearLayers];
  int hd[kLinearLayers];
  int nlayers;
  int64_t rows;
  int K;
};

// LDS of the kernel below: the x tile, or what takes its place (128 weight rows and the
// output chunk), whichever is larger
constexpr int linear_fwd_lds_bytes(int kd, int es) {
  const int xbytes = 256 * (kd + 8) * es, cbytes = 128 * (kd + 8) * es + 256 * (32 + 8) * es;
  return xbytes > cbytes ? xbytes : cbytes;
}

template <typename T, int KD>
__global__ __launch_bounds__(256) void linear_fwd_kernel(const LinearFwdArgs a) {
  using E = Elem<T>;
  using frag = typename E::frag;
  using vec = typename E::vec;
  constexpr int KS = KD / 16;        // MFMA steps over K
  constexpr int RT = 2, ROWS = 256;
  constexpr int LDX = KD + 8;        // padded row of the x tile and of a weight chunk
  constexpr int LDO = 32 + 8;        // padded row of an output chunk
  constexpr int XP = ROWS * KD / 8 / 256;  // 16-byte pieces of the x tile per lane
  // LDS: first the x tile; once its fragments are in registers, a group of weight rows and
  // the output chunk take its place
  extern __shared__ __attribute__((aligned(16))) unsigned char lin_smem[];
  T (*xs)[LDX] = reinterpret_cast<T (*)[LDX]>(lin_smem);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int cl = lane & 31, g = lane >> 5;
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;
  const T* xg = reinterpret_cast<const T*>(a.x);

  // x tile -> LDS -> registers
#pragma unroll
  for (int x4 = 0; x4 < XP; x4 += 4) {
    vec v[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int q = (x4 + x) * 256 + tid, r = q / (KD / 8), col = 8 * (q % (KD / 8));
      v[x] = vec{};
      if (row0 + r < a.rows) v[x] = *reinterpret_cast<const vec*>(xg + (row0 + r) * KD + col);
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const int q = (x4 + x) * 256 + tid, r = q / (KD / 8), col = 8 * (q % (KD / 8));
      *reinterpret_cast<vec*>(&xs[r][col]) = v[x];
    }
  }
  __syncthreads();
  frag xf[RT][KS];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int s = 0; s < KS; ++s) xf[t][s] = *reinterpret_cast<const frag*>(&xs[64 * wave + 32 * t + cl][16 * s + 8 * g]);
  __syncthreads();

  // The weights pass through LDS in groups of up to 128 output columns (four chunks of 32): the
  // next group waits in registers while this one is used, and takes its place between two
  // barriers.  (Loads and stores share one counter of operations in flight, and a wait for a
  // load is in effect a wait for the stores issued before it: staging every chunk of 32
  // columns separately made each chunk wait for the output stores of the one before.)
  constexpr int GROUP = 128;
  constexpr int GP = GROUP * KD / 8 / 256;  // 16-byte pieces of a group per lane
  int total = 0;
  for (int p = 0; p < a.nlayers; ++p) total += (a.n[p] + GROUP - 1) / GROUP;
  struct Cursor {
    int p, c;  // layer, group of 128 columns inside it
  };
  auto advance = [&](Cursor& cur) {
    if (GROUP * (cur.c + 1) < a.n[cur.p]) ++cur.c;
    else { ++cur.p; cur.c = 0; }
  };
  T (*wg)[LDX] = reinterpret_cast<T (*)[LDX]>(lin_smem);                              // [GROUP][LDX]
  T (*os)[LDO] = reinterpret_cast<T (*)[LDO]>(lin_smem + GROUP * LDX * sizeof(T));      // [ROWS][LDO]
  static_assert(GROUP * LDX * sizeof(T) + ROWS * LDO * sizeof(T) <= linear_fwd_lds_bytes(KD, (int)sizeof(T)), "the launcher sizes LDS with linear_fwd_lds_bytes");
  // rows GROUP c .. GROUP c + 127 of W_p (rows past N_p are zero)
  vec wr[GP];
  auto load_group = [&](const Cursor& cur) {
    const T* wsrc = reinterpret_cast<const T*>(a.w[cur.p]);
    const int N = a.n[cur.p];
#pragma unroll
    for (int x = 0; x < GP; ++x) {
      const int q = x * 256 + tid, r = q / (KD / 8), col = 8 * (q % (KD / 8));
      vec v = {};
      if (GROUP * cur.c + r < N) v = *reinterpret_cast<const vec*>(wsrc + (int64_t)(GROUP * cur.c + r) * KD + col);
      wr[x] = v;
    }
  };
  auto store_group = [&] {
#pragma unroll
    for (int x = 0; x < GP; ++x) {
      const int q = x * 256 + tid, r = q / (KD / 8), col = 8 * (q % (KD / 8));
      *reinterpret_cast<vec*>(&wg[r][col]) = wr[x];
    }
  };

  Cursor ld{0, 0}, use{0, 0};
  load_group(ld);
  advance(ld);
  for (int gq = 0; gq < total; ++gq) {
    store_group();
    __syncthreads();
    if (gq + 1 < total) { load_group(ld); advance(ld); }
    const int N = a.n[use.p];
    const T* bias = reinterpret_cast<const T*>(a.bias[use.p]);
    T* y = reinterpret_cast<T*>(a.y[use.p]);
    const int hd = a.hd[use.p];
    const int chunks = min(GROUP, N - GROUP * use.c + 31) / 32;  // chunks of 32 columns in this group
    for (int c = 0; c < chunks; ++c) {
      const int n0 = GROUP * use.c + 32 * c;
      // this lane's 16 columns of the chunk: n0 + 8 q4 + 4 g + e
      f32x16 acc[RT];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + 8 * (v / 4) + 4 * g + (v % 4);
        const float bv = (bias && n < N) ? (float)bias[n] : 0.f;
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[t][v] = bv;
      }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const frag af = *reinterpret_cast<const frag*>(&wg[32 * c + cl][16 * s + 8 * g]);
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[t] = E::mfma(af, xf[t][s], acc[t]);
      }
      // the chunk of this wave's 64 rows -> its own rows of the output tile -> global memory
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          typename E::vec4 ov;
#pragma unroll
          for (int e = 0; e < 4; ++e) ov[e] = (T)acc[t][4 * q4 + e];
          *reinterpret_cast<typename E::vec4*>(&os[64 * wave + 32 * t + cl][8 * q4 + 4 * g]) = ov;
        }
      // (the wave reads back only what it wrote: LDS operations of a wave complete in order)
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int idx = x * 64 + lane, r = 64 * wave + idx / 4, col = n0 + 8 * (idx % 4);
        const int64_t row = row0 + r;
        const vec v = *reinterpret_cast<const vec*>(&os[r][8 * (idx % 4)]);
        if (row < a.rows && col < N) {
          T* dst = y + linear_offset(row, col, N, hd, a.rows);
          if ((N % 8) == 0) {
            *reinterpret_cast<vec*>(dst) = v;
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (col + e < N) dst[e] = v[e];
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    advance(use);
    __syncthreads();  // every wave is done with this group's weights
  }
}

inline bool linear_fwd_k_ok(int64_t k) { return k == 32 || k == 64 || k == 128; }

template <typename T, int KD>
inline hipError_t linear_fwd_launch_k(const LinearFwdArgs& a, hipStream_t st) {
  const dim3 grid((unsigned)((a.rows + 255) / 256)), block(256);
  constexpr int lds = linear_fwd_lds_bytes(KD, (int)sizeof(T));
  if (lds > 64 * 1024) {
    // (more dynamic LDS than the default limit: raised once per kernel and device)
    const hipError_t e = raise_lds_limit(reinterpret_cast<const void*>(linear_fwd_kernel<T, KD>), lds);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL((linear_fwd_kernel<T, KD>), grid, block, lds, st, a);
  return hipGetLastError();
}

template <typename T>
inline hipError_t linear_fwd_launch_t(const LinearFwdArgs& a, hipStream_t st) {
  switch (a.K) {
    case 32: return linear_fwd_launch_k<T, 32>(a, st);
    case 64: return linear_fwd_launch_k<T, 64>(a, st);
    case 128: return linear_fwd_launch_k<T, 128>(a, st);
  }
  return hipErrorInvalidConfiguration;
}

}  // namespace tri
