// Kernel argument blocks shared by the launchers and the kernels.
#pragma once
#include <stdint.h>

namespace tri {

// strides are in elements; the last (d) stride of q/k/v/do is 1
struct Str5 { int64_t b, h, i, j; };   // [b, h, i, j, d], d contiguous

struct MaskPrepArgs {
  const uint8_t* mask;       // [b, n, n] bytes, nonzero = masked out
  int64_t sb, si, sk;
  uint32_t* keep;            // [b, n, nwords]: bit set = key is attended to
  uint32_t* rowflag;         // [b, n]: 1 = every valid key of the row is masked
  int n, nwords;
};

// The bias is re-tiled once per call into the exact register layout the kernels
// consume, zero-padded to whole 32 x 32 tiles, so that every wave-level load is
// one contiguous 1 KiB read with no bounds or alignment cases:
//   pack[((((bh*NP + jt)*NP + kt)*2 + r)*64 + lane)*8 + e]
//   packq (lane owns a query): bias[32 jt + lane%32][32 kt + 16 r + 8 (lane/32) + e]
//   packk (lane owns a key):   bias[32 jt + 16 r + 8 (lane/32) + e][32 kt + lane%32]
struct BiasPrepArgs {
  const void* bias;          // [b, h, n, n], any strides
  int64_t sb, sh, sj, sk;
  void* packq;               // may be null
  void* packk;               // may be null
  int H, N, NP;
};

// Split of the pre-pass grid: workgroups [0, bias_blocks) re-tile the bias
// (bias_blocks_per_head per batch*head), the rest take four mask rows each.
struct PrepGrid {
  unsigned bias_blocks, bias_blocks_per_head;
  int64_t mask_rows;         // b * n
};

struct FwdArgs {
  const void *q, *k, *v;
  const void* packq;
  const uint32_t* keep;
  const uint32_t* rowflag;
  void* o;
  float* lse;
  Str5 sq, sk, sv;
  int H, N, NP, nwords;
  float c;                   // log2(e) / sqrt(d): raw score -> log2 domain
  float sqrt_d;              // bias multiplier into the raw-score domain
  float neg_inf;             // finfo(dtype).min, reported in lse of fully masked rows
};

struct BwdArgs {
  const void *q, *k, *v, *o, *dout;
  const void *packq, *packk;
  const float* lse;
  const uint32_t* keep;
  const uint32_t* rowflag;
  // [b*h, n, n] 32-bit workspaces indexed [i, j], written by the dq kernel for the
  // other two: the per-query terms of the backward as rank-1 MFMA operand words
  // (see split_word): delta = -rowsum(o * do); lse2 = -lse * sqrt(d), the
  // log-sum-exp in the raw-score domain (ln n instead of lse for fully masked rows)
  uint32_t* delta;
  uint32_t* lse2;
  float* dbpart;             // [nchunks, b*h, n, n] fp32 partial db (nchunks > 1 only)
  void *dq, *dk, *dv, *db;
  Str5 sq, sk, sv, sdo;
  Str5 sdq, sdk, sdv;        // element strides of the gradients (d stride 1)
  int64_t sdb_b, sdb_h, sdb_j, sdb_k;  // element strides of db [b, h, j, k]
  int H, N, NP, nwords;
  int BH;                    // b * h
  int nchunks, rows_per_chunk;  // db kernel: split of the pair rows over workgroups
  float c;                   // log2(e) / sqrt(d)
  float sqrt_d;
  float scale;               // 1 / sqrt(d)
  // row-resident kernel run in several passes over the keys (rows longer than one pass holds)
  int key_tile0;             // first 32-key tile of this pass
  int pass_flags;            // 1: not the first pass, 2: not the last pass
  void* dq_lo;               // [b*h, n, n, d]: between passes dq is kept as dq (high part) + dq_lo
};

}  // namespace tri
