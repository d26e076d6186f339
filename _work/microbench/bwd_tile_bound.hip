// Issue-rate bounds of one backward tile on gfx950, registers only.
//
// One loop iteration is the instruction mix a backward kernel needs per 32 x 32 score
// tile at head dim 32 in bf16, with the additive terms already on the matrix pipe (bias
// as accumulator init, -lse and -delta through one extra MFMA each):
//   dq:     S (1 + 2 MFMAs), dP (1 + 2), 16 mul + 16 exp2, 16 mul (dS), 8 conversions, dq += dS K (2 MFMAs)
//   dk/dv:  S (1 + 2), dP (1 + 2), 16 mul + 16 exp2, 16 mul, 16 conversions (P and dS), dv (2) and dk (2) MFMAs
//   db:     S (1 + 2), dP (1 + 2), 16 mul + 16 exp2, 16 fma into the db accumulators
// The chains of tile t+1 are issued before the arithmetic of tile t, as in the kernels.
// No LDS, no global memory, no branches, no masks: the time per iteration per SIMD is a
// lower bound for the kernel's time per tile, whatever its tiling.
//
// build: hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//            -mllvm -amdgpu-mfma-vgpr-form=1 benchmark/microbench/bwd_tile_bound.hip -o bwd_tile_bound
// run:   ./bwd_tile_bound        (a few milliseconds of GPU time)
#include <hip/hip_runtime.h>
#include <cstdio>
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
#define ITERS 4096
#define MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)

__device__ inline bf16x8 pack8(const float* p) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    bf16x2 w = {(__bf16)p[2 * e], (__bf16)p[2 * e + 1]};
    r[2 * e] = w[0]; r[2 * e + 1] = w[1];
  }
  return r;
}

// KIND 0: dq, 1: dk/dv, 2: db
template <int KIND>
__global__ __launch_bounds__(256) void k(float* out, float seed, int iters) {
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed - i); }
  f32x16 sc, dp, sn, dn, bias, zero, acc0, acc1, acc2, acc3;
  for (int i = 0; i < 16; ++i) { sc[i] = seed * i; dp[i] = seed; zero[i] = 0.f; acc0[i] = acc1[i] = acc2[i] = acc3[i] = 0.f; bias[i] = seed * (i + threadIdx.x); }
  const float c = 0.25f;
  for (int it = 0; it < iters; ++it) {
    // chains of the next tile
    sn = MFMA(a, b, bias); sn = MFMA(b, a, sn); sn = MFMA(a, a, sn);
    dn = MFMA(b, b, zero); dn = MFMA(a, b, dn); dn = MFMA(b, a, dn);
    float p[16], ds[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) p[i] = __builtin_amdgcn_exp2f(sc[i] * c);
    if (KIND == 2) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc0[i] = __builtin_fmaf(p[i], dp[i], acc0[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) ds[i] = p[i] * dp[i];
      const bf16x8 d0 = pack8(ds), d1 = pack8(ds + 8);
      acc0 = MFMA(a, d0, acc0); acc0 = MFMA(b, d1, acc0);
      if (KIND == 1) {
        const bf16x8 p0 = pack8(p), p1 = pack8(p + 8);
        acc1 = MFMA(a, p0, acc1); acc1 = MFMA(b, p1, acc1);
      }
    }
    sc = sn; dp = dn;
    { u32x4 t = __builtin_bit_cast(u32x4, a); asm volatile("" : "+v"(t)); a = __builtin_bit_cast(bf16x8, t); }  // opaque: nothing is hoisted
  }
  float sum = 0.f;
  for (int i = 0; i < 16; ++i) sum += acc0[i] + acc1[i] + acc2[i] + acc3[i] + sc[i] + dp[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}

template <int KIND> void run(int wps) {
  float* out;
  if (hipMalloc(&out, 256 * 16 * 256 * sizeof(float)) != hipSuccess) { printf("hipMalloc failed\n"); return; }
  hipEvent_t s, e;
  (void)hipEventCreate(&s); (void)hipEventCreate(&e);
  const int blocks = 256 * wps;
  k<KIND><<<blocks, 256>>>(out, 0.001f, ITERS); (void)hipDeviceSynchronize();
  (void)hipEventRecord(s);
  k<KIND><<<blocks, 256>>>(out, 0.001f, ITERS);
  (void)hipEventRecord(e); (void)hipEventSynchronize(e);
  float ms; (void)hipEventElapsedTime(&ms, s, e);
  const char* names[] = {"dq", "dk/dv", "db"};
  printf("%-5s waves/SIMD=%d: %.3f ms  %.1f ns per tile per SIMD\n", names[KIND], wps, ms, ms * 1e6 / ITERS / wps);
  (void)hipFree(out);
}

int main() {
  for (int w : {1, 2, 3, 4}) run<0>(w);
  for (int w : {1, 2, 3, 4}) run<1>(w);
  for (int w : {1, 2, 3, 4}) run<2>(w);
  return 0;
}
