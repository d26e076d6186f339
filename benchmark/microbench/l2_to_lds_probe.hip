// How fast can a compute unit of the MI355X pull bytes that sit in its XCD's L2?
//
// One workgroup per compute unit (256 of them, 16 or 4 waves each) streams rows of 32 KiB
// (what the db kernel loads per pair row and 128 x 128 block: 2 KiB per wave) from a window of
// global memory that the workgroups of an XCD share and that fits its L2 (default 2 MiB per
// XCD, read round and round), either straight into LDS (global_load_lds_dwordx4, as the kernels
// do) or into registers (global_load_dwordx4).  Loads run `DEPTH` rows ahead; a row ends with
// a counted wait and (LDS variant) a barrier, like the ring of row buffers in the db kernel.
// Nothing is computed.  The program prints GB/s per compute unit and in total for several
// depths, and the same for a window that does not fit any cache (HBM).
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 benchmark/microbench/l2_to_lds_probe.hip -o /tmp/l2_to_lds_probe && /tmp/l2_to_lds_probe
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      std::printf("%s failed: %s\n", #x, hipGetErrorString(e_));                  \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// WAVES waves per workgroup; every wave loads LPW KiB per row (LPW wave loads of 1 KiB).
template <int WAVES, int LPW, int DEPTH, bool TO_LDS>
__global__ __launch_bounds__(WAVES * 64) void stream_kernel(const unsigned char* src, int64_t window_bytes, int rows, uint32_t* sink) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int ROW = WAVES * LPW * 1024;  // bytes of a row
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  // the workgroups of an XCD share one window; each starts at its own row of it
  const unsigned char* win = src + (int64_t)xcd * window_bytes;
  const int64_t rows_in_window = window_bytes / ROW;
  int64_t r = (int64_t)slot * 7 % rows_in_window;
  u32x4 acc[LPW] = {};
  u32x4 inflight[DEPTH > 0 ? DEPTH : 1][LPW];
  auto issue = [&](int buf) {
    const unsigned char* row = win + r * ROW + (int64_t)wave * LPW * 1024;
    r = r + 1 == rows_in_window ? 0 : r + 1;
#pragma unroll
    for (int x = 0; x < LPW; ++x) {
      if constexpr (TO_LDS) {
        const uint32_t dst = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)(smem + (buf * ROW + (wave * LPW + x) * 1024)));
        const uint32_t voff = (uint32_t)(x * 1024 + lane * 16);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst), "v"(voff), "s"(row) : "memory", "m0");
      } else {
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(inflight[buf][x]) : "v"((uint32_t)(x * 1024 + lane * 16)), "s"(row) : "memory");
      }
    }
  };
  constexpr int NBUF = DEPTH + 1;
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) issue(u);
  for (int q = 0; q < rows; q += NBUF) {
#pragma unroll
    for (int u = 0; u < NBUF; ++u) {
      issue((u + DEPTH) % NBUF);
      // everything but the newest DEPTH rows has landed
      asm volatile("s_waitcnt vmcnt(%0)" : : "n"(DEPTH * LPW) : "memory");
      if constexpr (TO_LDS) {
        asm volatile("s_barrier" ::: "memory");
      } else {
#pragma unroll
        for (int x = 0; x < LPW; ++x) acc[x] ^= inflight[u][x];
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if constexpr (TO_LDS) {
    __syncthreads();
    if (sink && threadIdx.x == 0) sink[blockIdx.x] = *reinterpret_cast<uint32_t*>(smem);
  } else {
    uint32_t x = 0;
#pragma unroll
    for (int k = 0; k < LPW; ++k) x ^= acc[k][0] ^ acc[k][1] ^ acc[k][2] ^ acc[k][3];
    if (sink && x == 0x12345u) sink[blockIdx.x] = x;
  }
}

template <int WAVES, int LPW, int DEPTH, bool TO_LDS>
int run(const char* name, const unsigned char* src, int64_t window_bytes, uint32_t* sink) {
  constexpr int ROW = WAVES * LPW * 1024;
  const int rows = 4096 / (DEPTH + 1) * (DEPTH + 1);
  const int lds = TO_LDS ? (DEPTH + 1) * ROW : 0;
  auto kernel = stream_kernel<WAVES, LPW, DEPTH, TO_LDS>;
  if (lds > 64 * 1024) CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 4; ++rep) {
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL(kernel, dim3(256), dim3(WAVES * 64), lds, 0, src, window_bytes, rows, sink);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (rep > 0 && ms < best) best = ms;
  }
  const double bytes = 256.0 * rows * ROW;
  std::printf("%-34s window/XCD %6.1f MiB  depth %d  row %2d KiB: %7.3f ms  %6.1f GB/s per CU  %5.2f TB/s total\n", name, window_bytes / 1048576.0, DEPTH,
              ROW / 1024, best, bytes / best / 1e6 / 256, bytes / best / 1e9);
  return 0;
}

int main() {
  const int64_t big = (int64_t)8 * 512 * 1048576;  // 512 MiB per XCD window: no cache holds it
  unsigned char* src = nullptr;
  uint32_t* sink = nullptr;
  CHECK(hipMalloc(&src, big));
  CHECK(hipMemset(src, 1, big));
  CHECK(hipMalloc(&sink, 4096));
  const int64_t l2 = 2 * 1048576, hbm = 512 * (int64_t)1048576;
  if (run<16, 2, 1, true>("16 waves -> LDS", src, l2, sink)) return 1;
  if (run<16, 2, 2, true>("16 waves -> LDS", src, l2, sink)) return 1;
  if (run<16, 2, 3, true>("16 waves -> LDS", src, l2, sink)) return 1;
  if (run<16, 2, 3, false>("16 waves -> registers", src, l2, sink)) return 1;
  if (run<16, 2, 7, false>("16 waves -> registers", src, l2, sink)) return 1;
  if (run<4, 8, 3, true>("4 waves -> LDS", src, l2, sink)) return 1;
  if (run<4, 8, 3, false>("4 waves -> registers", src, l2, sink)) return 1;
  if (run<16, 2, 3, true>("16 waves -> LDS (HBM)", src, hbm, sink)) return 1;
  if (run<16, 2, 3, false>("16 waves -> registers (HBM)", src, hbm, sink)) return 1;
  if (run<4, 8, 3, true>("4 waves -> LDS (HBM)", src, hbm, sink)) return 1;
  if (run<16, 2, 3, true>("16 waves -> LDS, 256 KiB window", src, 262144, sink)) return 1;
  return 0;
}
