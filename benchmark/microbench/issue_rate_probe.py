"""Issue-rate probes for gfx950: prints a HIP program whose kernels are loops over asm bodies.

Each kernel runs one instruction pattern 2000 times per wave, registers only (no memory, no
LDS, no branches inside the body), with independent operands rotated over 16 registers, on
256 workgroups of 4 or 8 waves (one or two waves per SIMD, two workgroups for twice that).
The program prints, per pattern and occupancy, the time per body from HIP events and the
clocks per body from the wave's own cycle counter.

pattern tokens: M = v_mfma_f32_32x32x16_bf16 (four accumulators in turn), m = v_mfma_f32_16x16x32_bf16,
F = v_fma_f32, U = v_mul_f32, E = v_exp_f32, C = v_cvt_pk_bf16_f32, D = v_dot2c_f32_bf16.
"split_a|b" patterns give waves 0-3 of a workgroup of 8 the body a and waves 4-7 the body b
(one wave of each kind per SIMD).

    python3 benchmark/microbench/issue_rate_probe.py > /tmp/issue_rate_probe.hip
    hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops /tmp/issue_rate_probe.hip -o /tmp/issue_rate_probe
    /tmp/issue_rate_probe
"""
import sys
pats = {}
def add(name, a, b=None): pats[name] = (a, b if b is not None else a)
add("M8", "M" * 8)
add("m16", "m" * 16)
add("F64", "F" * 64)
add("E64", "E" * 64)
add("C64", "C" * 64)
add("U64", "U" * 64)
for k in (1, 2, 3, 4, 6, 8, 12, 16):
    add(f"M1F{k}x8", ("M" + "F" * k) * 8)
for k in (2, 4, 8):
    add(f"M1E{k}x8", ("M" + "E" * k) * 8)
for k in (2, 4, 8):
    add(f"m1F{k}x16", ("m" + "F" * k) * 16)
add("E1F3x16", ("E" + "F" * 3) * 16)
add("E1F1x32", ("EF") * 32)
add("E1F7x8", ("E" + "F" * 7) * 8)
# two roles: waves 0-3 run a, waves 4-7 run b (one of each per SIMD)
add("split_M8|F64", "M" * 8, "F" * 64)
add("split_M8|E64", "M" * 8, "E" * 64)
add("split_F64|E64", "F" * 64, "E" * 64)
add("split_M8|C64", "M" * 8, "C" * 64)
add("split_M8|F32", "M" * 8, "F" * 32)
add("split_M8|F16", "M" * 8, "F" * 16)
# kernel-like mixes per tile
add("fwdmix", "MM" + "F" * 16 + "E" * 16 + "C" * 8 + "D" * 8 + "MM")
add("fwdmix_il", "".join("M" + "FFFF" + "EEEE" + "CC" + "DD" for _ in range(4)))
add("rowmix12", "".join("M" + "UU" + "E" + "U" + "C" for _ in range(12)) + "UUUU" + "EEEE" + "UUUU" + "CCCC")
add("rowmix10", "".join("M" + "UUU" + "EE" + "UUU" + "CC"  for _ in range(10))[: None])

def body(p):
    out = []; nm = nf = 0
    for ch in p:
        if ch == "M":
            out.append(f"v_mfma_f32_32x32x16_bf16 %{nm % 4}, %4, %5, %{nm % 4}"); nm += 1
        elif ch == "m":
            out.append(f"v_mfma_f32_16x16x32_bf16 %{6 + nm % 4}, %4, %5, %{6 + nm % 4}"); nm += 1
        else:
            r = 10 + nf % 16; r2 = 10 + (nf + 5) % 16; nf += 1
            if ch == "F": out.append(f"v_fma_f32 %{r}, %{r}, %26, %27")
            elif ch == "U": out.append(f"v_mul_f32 %{r}, %{r}, %26")
            elif ch == "E": out.append(f"v_exp_f32 %{r}, %{r}")
            elif ch == "C": out.append(f"v_cvt_pk_bf16_f32 %{r}, %{r}, %{r2}")
            elif ch == "D": out.append(f"v_dot2c_f32_bf16 %{r}, %26, %27")
    return "\\n".join(out)

print(r'''#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstring>
#include <cstdlib>
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
#define OPS "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3), "+v"(a), "+v"(b), "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3), \
  "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7]), "+v"(f[8]), "+v"(f[9]), \
  "+v"(f[10]), "+v"(f[11]), "+v"(f[12]), "+v"(f[13]), "+v"(f[14]), "+v"(f[15]), "+v"(k1), "+v"(k2)
#define SETUP \
  f32x16 c0, c1, c2, c3; f32x4 d0, d1, d2, d3; bf16x8 a, b; float f[16]; float k1 = 1.0f, k2 = 0.0f; \
  for (int i = 0; i < 16; ++i) { c0[i] = c1[i] = c2[i] = c3[i] = 0.f; f[i] = seed * i; } \
  for (int i = 0; i < 4; ++i) { d0[i] = d1[i] = d2[i] = d3[i] = 0.f; } \
  for (int i = 0; i < 8; ++i) { a[i] = (__bf16)0.f; b[i] = (__bf16)0.f; }
#define FINISH float s = 0; for (int i = 0; i < 16; ++i) s += f[i] + c0[i] + c1[i] + c2[i] + c3[i]; \
  for (int i = 0; i < 4; ++i) s += d0[i] + d1[i] + d2[i] + d3[i]; \
  if (s == 12345.f) out[threadIdx.x] = s;
''')
names = list(pats)
for i, n in enumerate(names):
    a, b = pats[n]
    print(f'''__global__ __launch_bounds__(512) void k{i}(float* out, float seed, int iters, long long* clk) {{
  SETUP
  long long t0 = __builtin_readcyclecounter();
  if (threadIdx.x < 256) {{
    for (int it = 0; it < iters; ++it) asm volatile("{body(a)}" : OPS);
  }} else {{
    for (int it = 0; it < iters; ++it) asm volatile("{body(b)}" : OPS);
  }}
  long long t1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0 && blockIdx.x == 0) clk[0] = t1 - t0;
  if (threadIdx.x == 256 && blockIdx.x == 0) clk[1] = t1 - t0;
  FINISH
}}''')
print('''struct K { const char* name; void (*fn)(float*, float, int, long long*); int na, nb; };
static K ks[] = {''')
for i, n in enumerate(names):
    a, b = pats[n]
    print(f'  {{"{n}", k{i}, {len(a)}, {len(b)}}},')
print(r'''};
int main(int argc, char** argv) {
  float* out; long long* clk;
  if (hipMalloc(&out, 4096) != hipSuccess || hipMalloc(&clk, 16) != hipSuccess) { printf("hipMalloc failed\n"); return 1; }
  hipEvent_t s, e; (void)hipEventCreate(&s); (void)hipEventCreate(&e);
  const int iters = 2000;
  for (auto& k : ks) {
    for (int threads : {256, 512}) for (int wgs : {1, 2}) {
      if (threads == 256 && strncmp(k.name, "split", 5) == 0) continue;
      if (threads == 512 && wgs == 2 && strncmp(k.name, "split", 5) != 0 && strstr(k.name, "mix") == nullptr) continue;
      int blocks = 256 * wgs;
      k.fn<<<blocks, threads>>>(out, 0.001f, 10, clk); (void)hipDeviceSynchronize();
      (void)hipEventRecord(s);
      k.fn<<<blocks, threads>>>(out, 0.001f, iters, clk);
      (void)hipEventRecord(e); (void)hipEventSynchronize(e);
      float ms; (void)hipEventElapsedTime(&ms, s, e);
      long long h[2]; (void)hipMemcpy(h, clk, 16, hipMemcpyDeviceToHost);
      int wps = threads / 256 * wgs;
      printf("%-16s waves/SIMD=%d (%dx%d): %.3f ms  %8.1f ns/body  clk/body wave0 %8.1f wave4 %8.1f  [%d|%d instr]\n", k.name, wps, wgs, threads / 64,
             ms, ms * 1e6 / iters, (double)h[0] / iters, threads == 512 ? (double)h[1] / iters : 0.0, k.na, k.nb);
      fflush(stdout);
    }
  }
  return 0;
}''')
