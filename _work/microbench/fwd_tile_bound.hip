// Issue-rate bound of one forward tile on gfx950, registers only.
//
// One loop iteration is the instruction mix the forward kernel needs per 32 x 32 score
// tile at head dim 32 in bf16: 2 score MFMAs (one chain), 16 fma, 16 exp2, 8 conversions
// to packed bf16, 8 dot2 row-sum steps, 2 P.V MFMAs (one chain), software pipelined like
// the kernel (the score MFMAs of tile t+1 are issued before the softmax arithmetic of
// tile t).  No LDS, no global memory, no branches, no masks, no bias conversion: the
// time per iteration per SIMD is a lower bound for the kernel's time per tile, whatever
// its tiling.  The variants switch groups of instructions off to show what each costs.
//
// build: hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//            -mllvm -amdgpu-mfma-vgpr-form=1 benchmark/microbench/fwd_tile_bound.hip -o fwd_tile_bound
// run:   ./fwd_tile_bound        (a few milliseconds of GPU time)
#include <hip/hip_runtime.h>
#include <cstdio>
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#define ITERS 4096
// one forward "tile" per iteration, registers only: 2 score MFMAs (chain), 16 fma, 16 exp2, 8 cvt_pk, 8 dot2c, 2 PV MFMAs (chain),
// software pipelined like the kernel: the score MFMAs of tile t+1 are issued before the softmax arithmetic of tile t.
// MODE bit0: MFMAs on (else a few adds), bit1: exp2 on (else a multiply), bit2: conversions and dot2 on (else plain adds)
template<int MODE>
__global__ __launch_bounds__(256) void k(float* out, float seed, int iters) {
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed - i); }
  f32x16 sc, sn, o, bias;
  for (int i = 0; i < 16; ++i) { sc[i] = seed * i; o[i] = 0.f; bias[i] = seed * (i + threadIdx.x); }
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  float l = 0.f; const float c = 0.25f, m = 1.0f;
  for (int it = 0; it < iters; ++it) {
    if (MODE & 1) { sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, bias, 0, 0, 0); sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, sn, 0, 0, 0); }
    else { sn = bias; for (int i = 0; i < 16; ++i) sn[i] += sc[i] * 1e-9f; }
    float p[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) { float x = __builtin_fmaf(sc[i], c, -m); p[i] = (MODE & 2) ? __builtin_amdgcn_exp2f(x) : x * 0.5f; }
    bf16x8 pf[2]; float ts = 0.f;
    if (MODE & 4) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          bf16x2 w = {(__bf16)p[8 * h + 2 * e], (__bf16)p[8 * h + 2 * e + 1]};
          pf[h][2 * e] = w[0]; pf[h][2 * e + 1] = w[1];
          ts = __builtin_amdgcn_fdot2_f32_bf16(w, ones, ts, false);
        }
      }
    } else {
      for (int h = 0; h < 2; ++h) for (int e = 0; e < 8; ++e) pf[h][e] = a[e];
      for (int i = 0; i < 16; ++i) ts += p[i];
    }
    l += ts;
    if (MODE & 1) { o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[0], o, 0, 0, 0); o = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, pf[1], o, 0, 0, 0); }
    else { for (int e = 0; e < 8; ++e) o[e] += (float)pf[0][e] + (float)pf[1][e]; }
    sc = sn;
    { typedef unsigned u32x4 __attribute__((ext_vector_type(4))); u32x4 t = __builtin_bit_cast(u32x4, a); asm volatile("" : "+v"(t)); a = __builtin_bit_cast(bf16x8, t); }  // opaque: nothing is hoisted, no data dependence
  }
  float sum = l; for (int i = 0; i < 16; ++i) sum += o[i] + sc[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}
template<int MODE> void run(int wps) {
  float* out;
  if (hipMalloc(&out, 256 * 16 * 256 * sizeof(float)) != hipSuccess) { printf("hipMalloc failed\n"); return; }
  hipEvent_t s, e;
  (void)hipEventCreate(&s); (void)hipEventCreate(&e);
  int blocks = 256 * wps;
  k<MODE><<<blocks, 256>>>(out, 0.001f, ITERS); (void)hipDeviceSynchronize();
  (void)hipEventRecord(s);
  k<MODE><<<blocks, 256>>>(out, 0.001f, ITERS);
  (void)hipEventRecord(e); (void)hipEventSynchronize(e);
  float ms; (void)hipEventElapsedTime(&ms, s, e);
  printf("mode mfma=%d exp=%d cvtdot=%d waves/SIMD=%d: %.3f ms  %.1f ns per tile per SIMD\n", MODE & 1, (MODE >> 1) & 1, (MODE >> 2) & 1, wps, ms, ms * 1e6 / ITERS / wps);
  (void)hipFree(out);
}
int main() {
  for (int w : {1, 2, 3, 4}) run<7>(w);
  for (int w : {2}) { run<5>(w); run<3>(w); run<1>(w); }
  return 0;
}
