#include <hip/hip_runtime.h>
#include <cstdio>
// Dependent-issue probes for gfx950: what it costs a wave to issue an instruction right behind
// the one that produces its operand.  The softmax arithmetic of one pair of scores is a chain
// (two fma, two exp2, one packed conversion, one row-sum step): the probes time eight such
// units written as tight chains, interleaved two and four at a time, and the chains alone.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         benchmark/microbench/dependent_issue_probe.hip -o /tmp/dependent_issue_probe && /tmp/dependent_issue_probe
#define LOOP(BODY) for (int it = 0; it < iters; ++it) asm volatile(BODY : "+v"(a0),"+v"(a1),"+v"(a2),"+v"(a3),"+v"(a4),"+v"(a5),"+v"(a6),"+v"(a7),"+v"(b0),"+v"(b1),"+v"(b2),"+v"(b3),"+v"(acc0),"+v"(acc1),"+v"(c),"+v"(m));
#define U_TIGHT(x0,x1,w,acc) "v_fma_f32 " x0 ", " x0 ", %14, %15\n v_fma_f32 " x1 ", " x1 ", %14, %15\n v_exp_f32 " x0 ", " x0 "\n v_exp_f32 " x1 ", " x1 "\n s_nop 0\n v_cvt_pk_bf16_f32 " w ", " x0 ", " x1 "\n v_dot2c_f32_bf16 " acc ", " w ", " w "\n"
template<int MODE> __global__ __launch_bounds__(256) void k(float* out, float seed, int iters, long long* clk) {
  float a0=seed,a1=seed*2,a2=seed*3,a3=seed*4,a4=seed*5,a5=seed*6,a6=seed*7,a7=seed*8,b0=0,b1=0,b2=0,b3=0,acc0=0,acc1=0,c=0.5f,m=-1.f;
  long long t0 = __builtin_readcyclecounter();
  if (MODE == 0) {  // 8 units, each a tight chain, different registers per unit pair
    LOOP(U_TIGHT("%0","%1","%8","%12") U_TIGHT("%2","%3","%9","%13") U_TIGHT("%4","%5","%10","%12") U_TIGHT("%6","%7","%11","%13")
         U_TIGHT("%0","%1","%8","%12") U_TIGHT("%2","%3","%9","%13") U_TIGHT("%4","%5","%10","%12") U_TIGHT("%6","%7","%11","%13"))
  } else if (MODE == 1) {  // the same 8 units, interleaved four at a time
#define IL4 "v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %1, %1, %14, %15\n v_fma_f32 %2, %2, %14, %15\n v_fma_f32 %3, %3, %14, %15\n v_fma_f32 %4, %4, %14, %15\n v_fma_f32 %5, %5, %14, %15\n v_fma_f32 %6, %6, %14, %15\n v_fma_f32 %7, %7, %14, %15\n" \
 "v_exp_f32 %0, %0\n v_exp_f32 %1, %1\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3\n v_exp_f32 %4, %4\n v_exp_f32 %5, %5\n v_exp_f32 %6, %6\n v_exp_f32 %7, %7\n" \
 "v_cvt_pk_bf16_f32 %8, %0, %1\n v_cvt_pk_bf16_f32 %9, %2, %3\n v_cvt_pk_bf16_f32 %10, %4, %5\n v_cvt_pk_bf16_f32 %11, %6, %7\n" \
 "v_dot2c_f32_bf16 %12, %8, %8\n v_dot2c_f32_bf16 %13, %9, %9\n v_dot2c_f32_bf16 %12, %10, %10\n v_dot2c_f32_bf16 %13, %11, %11\n"
    LOOP(IL4 IL4)
  } else if (MODE == 2) {  // dependent fma chain, 48 long
#define F8 "v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n v_fma_f32 %0, %0, %14, %15\n"
    LOOP(F8 F8 F8 F8 F8 F8)
  } else if (MODE == 3) {  // dependent exp chain, 16 long
#define E8 "v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n v_exp_f32 %0, %0\n"
    LOOP(E8 E8)
  } else if (MODE == 4) {  // exp then dependent cvt, 16 pairs
#define EC "v_exp_f32 %0, %0\n s_nop 0\n v_cvt_pk_bf16_f32 %8, %0, %1\n"
    LOOP(EC EC EC EC EC EC EC EC EC EC EC EC EC EC EC EC)
  } else if (MODE == 5) {  // cvt then dependent dot2, 16 pairs
#define CD "v_cvt_pk_bf16_f32 %8, %0, %1\n v_dot2c_f32_bf16 %12, %8, %8\n"
    LOOP(CD CD CD CD CD CD CD CD CD CD CD CD CD CD CD CD)
  } else if (MODE == 6) {  // units interleaved two at a time
#define IL2(x0,x1,x2,x3,w0,w1) "v_fma_f32 " x0 ", " x0 ", %14, %15\n v_fma_f32 " x1 ", " x1 ", %14, %15\n v_fma_f32 " x2 ", " x2 ", %14, %15\n v_fma_f32 " x3 ", " x3 ", %14, %15\n" \
  "v_exp_f32 " x0 ", " x0 "\n v_exp_f32 " x1 ", " x1 "\n v_exp_f32 " x2 ", " x2 "\n v_exp_f32 " x3 ", " x3 "\n v_cvt_pk_bf16_f32 " w0 ", " x0 ", " x1 "\n v_cvt_pk_bf16_f32 " w1 ", " x2 ", " x3 "\n v_dot2c_f32_bf16 %12, " w0 ", " w0 "\n v_dot2c_f32_bf16 %13, " w1 ", " w1 "\n"
    LOOP(IL2("%0","%1","%2","%3","%8","%9") IL2("%4","%5","%6","%7","%10","%11") IL2("%0","%1","%2","%3","%8","%9") IL2("%4","%5","%6","%7","%10","%11"))
  }
  long long t1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0 && blockIdx.x == 0) clk[0] = t1 - t0;
  float s = a0+a1+a2+a3+a4+a5+a6+a7+b0+b1+b2+b3+acc0+acc1;
  if (s == 12345.f) out[threadIdx.x] = s;
}
template<int MODE> void run(const char* name, int n) {
  float* out; long long* clk; (void)hipMalloc(&out, 4096); (void)hipMalloc(&clk, 16);
  const int iters = 2000;
  for (int wgs : {1, 2}) {
    k<MODE><<<256 * wgs, 256>>>(out, 0.001f, 10, clk); (void)hipDeviceSynchronize();
    hipEvent_t s, e; (void)hipEventCreate(&s); (void)hipEventCreate(&e);
    (void)hipEventRecord(s); k<MODE><<<256 * wgs, 256>>>(out, 0.001f, iters, clk); (void)hipEventRecord(e); (void)hipEventSynchronize(e);
    float ms; (void)hipEventElapsedTime(&ms, s, e); long long h; (void)hipMemcpy(&h, clk, 8, hipMemcpyDeviceToHost);
    printf("%-28s waves/SIMD=%d: %7.1f ns/body  %7.1f clk/body (wave 0)  [%d instr]\n", name, wgs, ms * 1e6 / iters, (double)h / iters, n); fflush(stdout);
  }
}
int main() {
  run<0>("8 units tight", 48); run<6>("8 units interleaved by 2", 48); run<1>("8 units interleaved by 4", 48);
  run<2>("48 dependent fma", 48); run<3>("16 dependent exp", 16); run<4>("16x exp->cvt", 32); run<5>("16x cvt->dot2", 32);
  return 0;
}
