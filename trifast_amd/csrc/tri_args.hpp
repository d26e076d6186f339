// Kernel argument blocks shared by the launchers and the kernels.
#pragma once
#include <stdint.h>

namespace tri {

// strides are in elements; the last (d) stride of q/k/v/do is 1, the last (k)
// stride of bias is 1.
struct Str5 { int64_t b, h, i, j; };   // [b, h, i, j, d], d contiguous
struct Str4 { int64_t b, h, j; };      // bias [b, h, j, k], k contiguous

struct MaskPrepArgs {
  const uint8_t* mask;       // [b, n, n] bytes, nonzero = masked out
  int64_t sb, si, sk;
  uint32_t* keep;            // [b, n, nwords]: bit set = key is attended to
  uint8_t* rowflag;          // [b, n]: 1 = every valid key of the row is masked
  int n, nwords;
};

struct FwdArgs {
  const void *q, *k, *v, *bias;
  const uint32_t* keep;
  const uint8_t* rowflag;
  void* o;
  float* lse;
  Str5 sq, sk, sv;
  Str4 sbias;
  int H, N, nwords;
  int bias_vec_ok;           // bias rows 16-byte aligned: vector path allowed
  float c;                   // log2(e) / sqrt(d): raw score -> log2 domain
  float sqrt_d;              // bias multiplier into the raw-score domain
  float neg_inf;             // finfo(dtype).min, reported in lse of fully masked rows
};

struct BwdArgs {
  const void *q, *k, *v, *bias, *o, *dout;
  const float* lse;
  const uint32_t* keep;
  const uint8_t* rowflag;
  float* delta;              // [b*h, n, n] fp32 workspace, indexed [i, j]
  void *dq, *dk, *dv, *db;
  Str5 sq, sk, sv, sdo;
  Str4 sbias;
  int H, N, nwords;
  int bias_vec_ok;
  float c;                   // log2(e) / sqrt(d)
  float sqrt_d;
  float scale;               // 1 / sqrt(d)
};

}  // namespace tri
