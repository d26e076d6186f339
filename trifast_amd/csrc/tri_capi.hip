// C ABI of the triangle-attention library (see include/trifast_hip.h):
// argument checking, workspace carving, the mask pre-pass and the fixed launch
// order of the backward kernels.  Nothing here allocates device memory.
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <mutex>

#include "../../include/trifast_hip.h"
#include "tri_common.hpp"
#include "tri_launch.hpp"
#include "tri_gate.hpp"
#include "tri_linear.hpp"

namespace tri {

// ---------------------------------------------------------------------------
// The pre-passes: one launch of workgroups of four waves; the first `bias_blocks`
// workgroups re-tile the bias, the rest turn mask rows into bit words, one wave per row.
//
// Mask: bytes -> "keep" bit words + fully-masked-row flags.  A row whose valid keys are
// all masked follows the additive-mask semantics of reference
// src/trifast/equiv.py:49,59-62: all logits saturate to the same value, so the row
// attends uniformly to every key; its keep words are set to "all valid keys" and
// rowflag tells the kernels to drop the q.k and bias terms.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void mask_prep_row(const MaskPrepArgs& a, int64_t bi, int lane) {
  const int b = (int)(bi / a.n), i = (int)(bi % a.n);
  const uint8_t* row = a.mask + b * a.sb + i * a.si;
  uint32_t* out = a.keep + bi * a.nwords;
  bool any_kept = false;
  // (contiguous, 16-byte aligned rows: the 32 bytes of a word are two vector loads)
  const bool vec_rows = a.sk == 1 && (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  for (int w = lane; w < a.nwords; w += 64) {
    uint32_t bits = 0;
    if (vec_rows && 32 * w + 32 <= a.n) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + 32 * w + 16 * half);
#pragma unroll
        for (int t = 0; t < 16; ++t)
          if (((v[t / 4] >> (8 * (t % 4))) & 0xffu) == 0) bits |= 1u << (16 * half + t);
      }
    } else {
      for (int t = 0; t < 32; ++t) {
        const int key = 32 * w + t;
        if (key < a.n && row[key * a.sk] == 0) bits |= 1u << t;
      }
    }
    out[w] = bits;
    any_kept |= bits != 0;
  }
  const bool row_kept = __any(any_kept);
  if (!row_kept) {
    for (int w = lane; w < a.nwords; w += 64) {
      const int rem = a.n - 32 * w;
      out[w] = rem >= 32 ? 0xffffffffu : ((1u << rem) - 1u);
    }
  }
  if (lane == 0) a.rowflag[bi] = row_kept ? 0 : 1;
}

// Bias: re-tile bias[b, h, j, k] (any strides) into the register layouts of the kernels
// (see BiasPrepArgs), zero-padded to whole tiles.  One thread writes the 8 elements of
// one (tile, r, lane) slot of each requested layout.
template <typename T>
__device__ __forceinline__ void bias_prep_slot(const BiasPrepArgs& a, int bh, int64_t slot) {
  const int b = bh / a.H, h = bh % a.H;
  if (slot >= (int64_t)a.NP * a.NP * 128) return;  // ((jt*NP + kt)*2 + r)*64 + lane
  const int lane = slot & 63, r = (slot >> 6) & 1;
  const int tile = (int)(slot >> 7);
  const int jt = tile / a.NP, kt = tile % a.NP;
  const int l32 = lane & 31, g = lane >> 5;
  const T* src = reinterpret_cast<const T*>(a.bias) + b * a.sb + h * a.sh;
  const int64_t out = ((int64_t)bh * a.NP * a.NP * 128 + slot) * 8;
  typedef T tvec __attribute__((ext_vector_type(8)));
  if (a.packq) {
    T* dst = reinterpret_cast<T*>(a.packq) + out;
    const int j = 32 * jt + l32;
    const int key0 = 32 * kt + 16 * r + 8 * g;
    const T* p = src + j * a.sj + key0 * a.sk;
    // (eight consecutive keys of a row with contiguous keys: one vector load where it is aligned)
    if (a.sk == 1 && j < a.N && key0 + 8 <= a.N && (reinterpret_cast<uintptr_t>(p) & (sizeof(tvec) - 1)) == 0) {
      *reinterpret_cast<tvec*>(dst) = *reinterpret_cast<const tvec*>(p);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = (j < a.N && key0 + e < a.N) ? p[e * a.sk] : (T)0.f;
    }
  }
  if (a.packk) {
    T* dst = reinterpret_cast<T*>(a.packk) + out;
    const int key = 32 * kt + l32;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = 32 * jt + 16 * r + 8 * g + e;
      dst[e] = (j < a.N && key < a.N) ? src[j * a.sj + key * a.sk] : (T)0.f;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void prep_kernel(const MaskPrepArgs m, const BiasPrepArgs a, const PrepGrid g) {
  if (blockIdx.x < g.bias_blocks) {
    const unsigned bh = blockIdx.x / g.bias_blocks_per_head, bx = blockIdx.x % g.bias_blocks_per_head;
    bias_prep_slot<T>(a, (int)bh, (int64_t)bx * 256 + threadIdx.x);
  } else {
    const int64_t row = (int64_t)(blockIdx.x - g.bias_blocks) * 4 + (threadIdx.x >> 6);
    if (row < g.mask_rows) mask_prep_row(m, row, threadIdx.x & 63);
  }
}

hipError_t prep_launch(const MaskPrepArgs& m, int b, const BiasPrepArgs& a, int bh, int dtype, hipStream_t st) {
  const int64_t slots = (int64_t)a.NP * a.NP * 128;
  PrepGrid g;
  g.bias_blocks_per_head = (unsigned)((slots + 255) / 256);
  g.mask_rows = (int64_t)b * m.n;
  const int64_t bias_blocks = (int64_t)g.bias_blocks_per_head * bh, blocks = bias_blocks + (g.mask_rows + 3) / 4;
  if (blocks > 0x7fffffff) return hipErrorInvalidConfiguration;
  g.bias_blocks = (unsigned)bias_blocks;
  const dim3 grid((unsigned)blocks);
  switch (dtype) {
    case kF32: hipLaunchKernelGGL(prep_kernel<float>, grid, dim3(256), 0, st, m, a, g); break;
    case kBF16: hipLaunchKernelGGL(prep_kernel<__bf16>, grid, dim3(256), 0, st, m, a, g); break;
    default: hipLaunchKernelGGL(prep_kernel<_Float16>, grid, dim3(256), 0, st, m, a, g); break;
  }
  return hipGetLastError();
}

}  // namespace tri

// Scratch of trifast_fwd_static: device memory that lives in the library's code
// object, one copy per GPU, from load until the process ends.  The array's name is
// a host-side handle only; kernels and pre-passes get the device address that
// hipGetSymbolAddress returns for the current device (static_scratch below).
static __device__ __align__(256) unsigned char scratch[TRIFAST_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return (int)e > 0 ? (int)e : 1;
}

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(TRIFAST_EINVAL, "device %d is beyond the %d devices the static scratch table holds", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

int64_t align256(int64_t x) { return (x + 255) & ~int64_t(255); }
int elem_size(int dtype) { return dtype == TRIFAST_F32 ? 4 : 2; }

float dtype_min(int dtype) {
  switch (dtype) {
    case TRIFAST_BF16: return -3.3895313892515355e38f;
    case TRIFAST_F16: return -65504.0f;
    default: return -std::numeric_limits<float>::max();
  }
}

// workspace layout: keep words | row flags | packq | (backward only) packk | -delta | lse2 | db partials
struct Workspace {
  uint32_t* keep;
  uint32_t* rowflag;
  void* packq;
  void* packk;
  uint32_t* delta;
  uint32_t* lse2;
  float* dbpart;
  int nwords, np;
};

int64_t ws_mask_bytes(int64_t b, int64_t n) {
  const int64_t nwords = (n + 31) / 32;
  return align256(b * n * nwords * 4) + align256(b * n * 4);
}

int64_t ws_pack_bytes(int64_t b, int64_t h, int64_t n, int dtype) {
  const int64_t np = (n + 31) / 32;
  return align256(b * h * np * np * 1024 * elem_size(dtype));
}

Workspace carve(void* ws, int64_t b, int64_t h, int64_t n, int dtype) {
  Workspace w;
  const int64_t nwords = (n + 31) / 32;
  char* p = static_cast<char*>(ws);
  w.keep = reinterpret_cast<uint32_t*>(p);
  p += align256(b * n * nwords * 4);
  w.rowflag = reinterpret_cast<uint32_t*>(p);
  p += align256(b * n * 4);
  w.packq = p;
  p += ws_pack_bytes(b, h, n, dtype);
  w.packk = p;
  p += ws_pack_bytes(b, h, n, dtype);
  w.delta = reinterpret_cast<uint32_t*>(p);
  p += align256(b * h * n * n * 4);
  w.lse2 = reinterpret_cast<uint32_t*>(p);
  p += align256(b * h * n * n * 4);
  w.dbpart = reinterpret_cast<float*>(p);
  w.nwords = (int)nwords;
  w.np = (int)nwords;
  return w;
}

int check_common(int64_t b, int64_t h, int64_t n, int64_t d, int dtype) {
  if (b < 1 || h < 1 || n < 1) return fail(TRIFAST_EINVAL, "sizes must be positive (b=%lld h=%lld n=%lld)", (long long)b, (long long)h, (long long)n);
  if (dtype != TRIFAST_F32 && dtype != TRIFAST_BF16 && dtype != TRIFAST_F16) return fail(TRIFAST_EINVAL, "unknown dtype code %d", dtype);
  if (!tri::head_dim_ok((int)d)) return fail(TRIFAST_EUNSUPPORTED, "head dim %lld is not one of the compiled ones (16, 32, 64, 128)", (long long)d);
  // (b*h, padded to a multiple of 8, is a grid extent)
  if (n > 65535 || b * h > 65528) return fail(TRIFAST_EINVAL, "n must be at most 65535 and b*h at most 65528");
  return 0;
}

// q-like tensor: 16-byte aligned base, strides multiples of the vector width, d stride 1
int check_qlike(const char* name, const void* p, const int64_t* s, int dtype) {
  if (!p || !s) return fail(TRIFAST_EINVAL, "%s: null pointer", name);
  const int vec = 16 / elem_size(dtype);
  if (s[4] != 1) return fail(TRIFAST_EALIGN, "%s: last stride must be 1 (got %lld)", name, (long long)s[4]);
  if ((reinterpret_cast<uintptr_t>(p) & 15) != 0) return fail(TRIFAST_EALIGN, "%s: base pointer is not 16-byte aligned", name);
  for (int t = 0; t < 4; ++t)
    if (s[t] % vec != 0) return fail(TRIFAST_EALIGN, "%s: stride %d (%lld) is not a multiple of %d elements", name, t, (long long)s[t], vec);
  // the stage loads address the rows of a tile (up to 256 of them) with 32-bit byte offsets
  // from the tile's first row
  const int64_t max_row_stride = (int64_t(1) << 24) / elem_size(dtype);
  if (s[3] < 0 || s[3] >= max_row_stride)
    return fail(TRIFAST_EUNSUPPORTED, "%s: stride 3 (%lld) must be in [0, %lld) elements", name, (long long)s[3], (long long)max_row_stride);
  return 0;
}

tri::Str5 str5(const int64_t* s) { return tri::Str5{s[0], s[1], s[2], s[3]}; }

// contiguous [b, h, n, n, d] / [b, h, n, n] element strides, for outputs whose strides are not given
void contiguous5(int64_t* s, int64_t h, int64_t n, int64_t d) {
  s[4] = 1; s[3] = d; s[2] = n * d; s[1] = n * n * d; s[0] = h * n * n * d;
}
void contiguous4(int64_t* s, int64_t h, int64_t n) {
  s[3] = 1; s[2] = n; s[1] = n * n; s[0] = h * n * n;
}

// Both pre-passes in one launch: keep words and row flags of the mask, the packed bias.
int run_prep(const uint8_t* mask, const int64_t* ms, const void* bias, const int64_t* bs, const Workspace& w, bool want_k,
             int64_t b, int64_t h, int64_t n, int dtype, hipStream_t st) {
  tri::MaskPrepArgs m;
  m.mask = mask;
  m.sb = ms[0]; m.si = ms[1]; m.sk = ms[2];
  m.keep = w.keep;
  m.rowflag = w.rowflag;
  m.n = (int)n;
  m.nwords = w.nwords;
  tri::BiasPrepArgs p;
  p.bias = bias;
  p.sb = bs[0]; p.sh = bs[1]; p.sj = bs[2]; p.sk = bs[3];
  p.packq = w.packq;
  p.packk = want_k ? w.packk : nullptr;
  p.H = (int)h; p.N = (int)n; p.NP = w.np;
  hipError_t e = tri::prep_launch(m, (int)b, p, (int)(b * h), dtype, st);
  if (e != hipSuccess) return hip_fail(e, "mask and bias pre-pass launch");
  return 0;
}

}  // namespace

extern "C" {

int trifast_abi_version(void) { return TRIFAST_ABI_VERSION; }

const char* trifast_last_error(void) { return g_err; }

int trifast_device_clock_mhz(int device) {
  g_err[0] = 0;
  int count = 0, khz = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e == hipSuccess && (device < 0 || device >= count)) return fail(TRIFAST_EINVAL, "device clock: no device %d (%d visible)", device, count);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, device);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // the runtime keeps the error for the next caller otherwise
    hip_fail(e, "device clock");
    return TRIFAST_EINVAL;
  }
  return khz / 1000;
}

int trifast_num_tiles(int kernel) {
  switch (kernel) {
    case TRIFAST_KERNEL_FWD: return tri::fwd_num_tiles();
    case TRIFAST_KERNEL_BWD_Q: return tri::bwd_q_num_tiles();
    case TRIFAST_KERNEL_BWD_KV: return tri::bwd_kv_num_tiles();
    case TRIFAST_KERNEL_BWD_B: return tri::bwd_b_num_tiles();
  }
  return fail(TRIFAST_EINVAL, "unknown kernel id %d", kernel);
}

int trifast_tile_info(int kernel, int tile, int* block_j, int* block_k, int* num_waves) {
  const int nt = trifast_num_tiles(kernel);
  if (nt < 0) return nt;
  if (tile < 0 || tile >= nt) return fail(TRIFAST_EINVAL, "tile %d out of range for kernel %d", tile, kernel);
  tri::TileInfo t;
  switch (kernel) {
    case TRIFAST_KERNEL_FWD: t = tri::fwd_tile_info(tile); break;
    case TRIFAST_KERNEL_BWD_Q: t = tri::bwd_q_tile_info(tile); break;
    case TRIFAST_KERNEL_BWD_KV: t = tri::bwd_kv_tile_info(tile); break;
    default: t = tri::bwd_b_tile_info(tile); break;
  }
  if (block_j) *block_j = t.block_j;
  if (block_k) *block_k = t.block_k;
  if (num_waves) *num_waves = t.num_waves;
  return 0;
}

int trifast_supports(int kernel, int tile, int64_t n, int64_t h, int64_t d, int dtype) {
  (void)h;
  if (dtype != TRIFAST_F32 && dtype != TRIFAST_BF16 && dtype != TRIFAST_F16) return 0;
  switch (kernel) {
    case TRIFAST_KERNEL_FWD: return tri::fwd_supports(tile, n, (int)d, dtype) ? 1 : 0;
    case TRIFAST_KERNEL_BWD_Q: return tri::bwd_q_supports(tile, n, (int)d, dtype) ? 1 : 0;
    case TRIFAST_KERNEL_BWD_KV: return tri::bwd_kv_supports(tile, n, (int)d, dtype) ? 1 : 0;
    case TRIFAST_KERNEL_BWD_B: return tri::bwd_b_supports(tile, n, (int)d, dtype) ? 1 : 0;
  }
  return 0;
}

int trifast_default_tile(int kernel, int64_t n, int64_t h, int64_t d, int dtype) {
  (void)h;
  // Picks measured on MI355X (bf16/fp16 at d = 16, 32, 64 and fp32 at d = 32, 64), by
  // the bytes of one q/k/v row: the wider the row, the fewer pair rows and tiles per
  // wave fit in registers.  Anything that does not fit the shape falls back to tile 0
  // and then to the first tile that supports it.
  const int64_t row_bytes = d * elem_size(dtype);
  int pick = 0;
  switch (kernel) {
    case TRIFAST_KERNEL_FWD:
      // pair rows that share a bias tile: one for the smallest and the widest rows; two for
      // 128-byte rows (one in fp32) and for 64-byte 16-bit rows of fewer than 768 keys; four
      // above that, with the scheduled loop for workgroups without masked keys; 32-byte rows:
      // four, or two with 64 keys per stage from 256 keys on
      if (n <= 64 || row_bytes >= 256) pick = 0;
      else if (row_bytes == 128) pick = dtype == TRIFAST_F32 ? 0 : 4;
      else if (row_bytes == 64) pick = dtype == TRIFAST_F32 ? 3 : (n < 768 ? 4 : 7);  // (7: four rows, scheduled loop)
      else pick = n >= 256 ? 1 : 3;
      break;
    case TRIFAST_KERNEL_BWD_Q:  // 2 pair rows, 64 keys per stage; one row from 128-byte rows on
      pick = (n <= 64 || row_bytes >= 128) ? 0 : 1;
      break;
    case TRIFAST_KERNEL_BWD_KV:  // 2 pair rows, 32 queries per stage; one row, 64 queries for wide 16-bit rows
      pick = (n <= 64 || row_bytes >= 256 || (row_bytes == 128 && dtype != TRIFAST_F32)) ? 0 : 1;
      // 16-bit rows of up to 1024 keys at head dim 16 or 32, up to 384 keys at head dim 64 (more
      // of them spill): the row-resident tile that also produces dq, with as few key tiles per
      // wave as hold the row (ids follow the four streaming tiles).  It wins from the smallest
      // rows on, where it is one launch instead of two.
      if (dtype != TRIFAST_F32 && n <= 1024 && (d == 16 || d == 32 || (d == 64 && n <= 384))) pick = 4 + (n <= 256 ? 0 : (int)((n - 1) / 128) - 1);
      // longer rows of head dim 32: the same kernel in passes of 1024 keys
      if (d == 32 && dtype != TRIFAST_F32 && n > 1024 && n <= 8192) pick = tri::bwd_kv_num_tiles() - 1;
      break;
    case TRIFAST_KERNEL_BWD_B:
      // 64 x 64 block of 4 waves up to 256 keys (more workgroups than a larger block gives
      // there), for 32-byte rows and for the widest ones; else 128 x 128 of 16 waves, of 8 waves
      // for 128-byte rows
      pick = (n <= 256 || row_bytes <= 32 || row_bytes >= 256) ? 2 : (row_bytes == 128 ? 3 : 4);
      break;

    default: return fail(TRIFAST_EINVAL, "unknown kernel id %d", kernel);
  }
  if (!trifast_supports(kernel, pick, n, h, d, dtype)) pick = 0;
  if (!trifast_supports(kernel, pick, n, h, d, dtype)) {
    const int nt = trifast_num_tiles(kernel);
    for (int t = 0; t < nt; ++t)
      if (trifast_supports(kernel, t, n, h, d, dtype)) return t;
    return fail(TRIFAST_EUNSUPPORTED, "no tile of kernel %d supports n=%lld d=%lld dtype=%d", kernel, (long long)n, (long long)d, dtype);
  }
  return pick;
}

int trifast_bwd_kv_tile_writes_dq(int tile) { return tri::bwd_kv_tile_writes_dq(tile) ? 1 : 0; }

int64_t trifast_fwd_workspace_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int dtype) {
  (void)d;
  if (b < 1 || h < 1 || n < 1) return fail(TRIFAST_EINVAL, "sizes must be positive");
  return ws_mask_bytes(b, n) + ws_pack_bytes(b, h, n, dtype);
}

// The tail of the backward workspace serves two kernels that run one after the other: the
// low parts of dq between the passes of the row-resident kernel over a long row (where a tile
// of that kind supports the shape), then the db partials of the row chunks.
static int64_t ws_tail_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int dtype) {
  const int64_t chunks = tri::bwd_b_chunks(n, b * h, (int)d * elem_size(dtype));
  const int64_t parts = chunks > 1 ? align256(chunks * b * h * n * n * 4) : 0;
  const bool passes = tri::head_dim_ok((int)d) && tri::bwd_kv_supports(tri::bwd_kv_num_tiles() - 1, n, (int)d, dtype);
  const int64_t lo = passes ? align256(b * h * n * n * d * elem_size(dtype)) : 0;
  return parts > lo ? parts : lo;
}

int64_t trifast_bwd_workspace_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int dtype) {
  if (b < 1 || h < 1 || n < 1) return fail(TRIFAST_EINVAL, "sizes must be positive");
  return ws_mask_bytes(b, n) + 2 * ws_pack_bytes(b, h, n, dtype) + 2 * align256(b * h * n * n * 4) + ws_tail_bytes(b, h, n, d, dtype);
}

// Forward with the workspace either given by the caller or (use_static) taken from the
// library's own static scratch array.
static int fwd_impl(bool use_static, void* o, float* lse, const void* q, const void* k, const void* v, const void* bias,
                    const uint8_t* mask, int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                    const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                    const int64_t* bias_strides, const int64_t* mask_strides, int tile, void* workspace,
                    int64_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = check_common(b, h, n, d, dtype);
  if (rc) return rc;
  if (!o || !lse || !bias || !mask || !bias_strides || !mask_strides) return fail(TRIFAST_EINVAL, "null pointer argument");
  if ((rc = check_qlike("q", q, q_strides, dtype))) return rc;
  if ((rc = check_qlike("k", k, k_strides, dtype))) return rc;
  if ((rc = check_qlike("v", v, v_strides, dtype))) return rc;
  if ((reinterpret_cast<uintptr_t>(o) & 15) != 0) return fail(TRIFAST_EALIGN, "o: base pointer is not 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0) return fail(TRIFAST_EALIGN, "lse: base pointer is not 4-byte aligned");
  if (use_static) {
    const int64_t need = trifast_fwd_workspace_bytes(b, h, n, d, dtype);
    if (need > (int64_t)TRIFAST_STATIC_SCRATCH_BYTES)
      return fail(TRIFAST_EWORKSPACE, "trifast_fwd_static: this shape needs %lld bytes of scratch, the static array holds %lld "
                  "(use trifast_fwd with a caller-provided workspace)", (long long)need, (long long)TRIFAST_STATIC_SCRATCH_BYTES);
    if ((rc = static_scratch(&workspace))) return rc;
    workspace_bytes = TRIFAST_STATIC_SCRATCH_BYTES;
  }
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
      workspace_bytes < trifast_fwd_workspace_bytes(b, h, n, d, dtype))
    return fail(TRIFAST_EWORKSPACE, "workspace missing, misaligned or smaller than trifast_fwd_workspace_bytes");
  if (tile < 0) tile = trifast_default_tile(TRIFAST_KERNEL_FWD, n, h, d, dtype);
  if (tile < 0) return tile;
  if (!tri::fwd_supports(tile, n, (int)d, dtype)) return fail(TRIFAST_EUNSUPPORTED, "forward tile %d does not support n=%lld d=%lld dtype=%d", tile, (long long)n, (long long)d, dtype);

  hipStream_t st = static_cast<hipStream_t>(stream);
  const Workspace w = carve(workspace, b, h, n, dtype);
  if ((rc = run_prep(mask, mask_strides, bias, bias_strides, w, false, b, h, n, dtype, st))) return rc;

  tri::FwdArgs a;
  a.q = q; a.k = k; a.v = v; a.packq = w.packq;
  a.keep = w.keep; a.rowflag = w.rowflag;
  a.o = o; a.lse = lse;
  a.sq = str5(q_strides); a.sk = str5(k_strides); a.sv = str5(v_strides);
  a.H = (int)h; a.N = (int)n; a.NP = w.np; a.nwords = w.nwords;
  a.c = (float)(1.4426950408889634 / std::sqrt((double)d));
  a.sqrt_d = (float)std::sqrt((double)d);
  a.neg_inf = dtype_min(dtype);
  hipError_t e = tri::fwd_launch(a, (int)(b * h), (int)d, dtype, tile, st);
  if (e != hipSuccess) return hip_fail(e, "forward launch");
  return 0;
}

int trifast_fwd(void* o, float* lse, const void* q, const void* k, const void* v, const void* bias,
                const uint8_t* mask, int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                const int64_t* bias_strides, const int64_t* mask_strides, int tile, void* workspace,
                int64_t workspace_bytes, void* stream) {
  return fwd_impl(false, o, lse, q, k, v, bias, mask, b, h, n, d, dtype, q_strides, k_strides, v_strides,
                  bias_strides, mask_strides, tile, workspace, workspace_bytes, stream);
}

int trifast_fwd_static(void* o, float* lse, const void* q, const void* k, const void* v, const void* bias,
                       const uint8_t* mask, int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                       const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                       const int64_t* bias_strides, const int64_t* mask_strides, int tile, void* stream) {
  return fwd_impl(true, o, lse, q, k, v, bias, mask, b, h, n, d, dtype, q_strides, k_strides, v_strides,
                  bias_strides, mask_strides, tile, nullptr, 0, stream);
}

static int bwd_impl(int which, void* dq, void* dk, void* dv, void* db, const void* dout, const void* q,
                    const void* k, const void* v, const void* bias, const uint8_t* mask, const void* o,
                    const float* lse, int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                    const int64_t* do_strides, const int64_t* q_strides, const int64_t* k_strides,
                    const int64_t* v_strides, const int64_t* bias_strides, const int64_t* mask_strides,
                    const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                    const int64_t* db_strides,
                    const int* tiles, void* workspace, int64_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  int rc = check_common(b, h, n, d, dtype);
  if (rc) return rc;
  if (!bias || !mask || !o || !lse || !bias_strides || !mask_strides) return fail(TRIFAST_EINVAL, "null pointer argument");
  if ((rc = check_qlike("do", dout, do_strides, dtype))) return rc;
  if ((rc = check_qlike("q", q, q_strides, dtype))) return rc;
  if ((rc = check_qlike("k", k, k_strides, dtype))) return rc;
  if ((rc = check_qlike("v", v, v_strides, dtype))) return rc;
  if ((reinterpret_cast<uintptr_t>(o) & 15) != 0) return fail(TRIFAST_EALIGN, "o: base pointer is not 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(lse) & 3) != 0) return fail(TRIFAST_EALIGN, "lse: base pointer is not 4-byte aligned");
  const bool all = which < 0;
  bool do_q = all || which == TRIFAST_KERNEL_BWD_Q;
  const bool do_kv = all || which == TRIFAST_KERNEL_BWD_KV;
  const bool do_b = all || which == TRIFAST_KERNEL_BWD_B;
  if (!do_q && !do_kv && !do_b) return fail(TRIFAST_EINVAL, "kernel id %d is not a backward kernel", which);
  int tq = tiles ? tiles[0] : -1, tkv = tiles ? tiles[1] : -1, tb = tiles ? tiles[2] : -1;
  if (tq < 0) tq = trifast_default_tile(TRIFAST_KERNEL_BWD_Q, n, h, d, dtype);
  if (tkv < 0) tkv = trifast_default_tile(TRIFAST_KERNEL_BWD_KV, n, h, d, dtype);
  if (tb < 0) tb = trifast_default_tile(TRIFAST_KERNEL_BWD_B, n, h, d, dtype);
  if (tq < 0 || tkv < 0 || tb < 0) return TRIFAST_EUNSUPPORTED;
  // a row-resident dk/dv tile produces dq (and the per-query planes) as well: the dq
  // kernel is not launched with it, and dq must be given whenever it runs
  const bool kv_writes_dq = do_kv && tri::bwd_kv_tile_writes_dq(tkv);
  const bool need_dq = do_q || kv_writes_dq;
  if (all && kv_writes_dq) do_q = false;
  // gradients: the caller's strides, or contiguous when none are given
  int64_t c5[5], c4[4];
  contiguous5(c5, h, n, d);
  contiguous4(c4, h, n);
  if (!dq_strides) dq_strides = c5;
  if (!dk_strides) dk_strides = c5;
  if (!dv_strides) dv_strides = c5;
  if (!db_strides) db_strides = c4;
  if (need_dq && (rc = check_qlike("dq", dq, dq_strides, dtype))) return rc;
  if (do_kv && (rc = check_qlike("dk", dk, dk_strides, dtype))) return rc;
  if (do_kv && (rc = check_qlike("dv", dv, dv_strides, dtype))) return rc;
  if (do_b && !db) return fail(TRIFAST_EINVAL, "db: null pointer");
  // (db is written with 16-byte stores where its strides allow it)
  if (do_b && (reinterpret_cast<uintptr_t>(db) & 15) != 0) return fail(TRIFAST_EALIGN, "db: base pointer is not 16-byte aligned");

  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 ||
      workspace_bytes < trifast_bwd_workspace_bytes(b, h, n, d, dtype))
    return fail(TRIFAST_EWORKSPACE, "workspace missing, misaligned or smaller than trifast_bwd_workspace_bytes");

  if (do_q && !tri::bwd_q_supports(tq, n, (int)d, dtype)) return fail(TRIFAST_EUNSUPPORTED, "bwd_q tile %d unsupported for this shape", tq);
  if (do_kv && !tri::bwd_kv_supports(tkv, n, (int)d, dtype)) return fail(TRIFAST_EUNSUPPORTED, "bwd_kv tile %d unsupported for this shape", tkv);
  if (do_b && !tri::bwd_b_supports(tb, n, (int)d, dtype)) return fail(TRIFAST_EUNSUPPORTED, "bwd_b tile %d unsupported for this shape", tb);

  hipStream_t st = static_cast<hipStream_t>(stream);
  const Workspace w = carve(workspace, b, h, n, dtype);
  // The pre-passes are cheap (n^2 elements) and make every single-kernel call
  // self-contained, so they run on every call.
  // (only the dk/dv tiles that do not also produce dq read the key-major packed bias)
  const bool want_k = do_kv && !tri::bwd_kv_tile_writes_dq(tkv);
  if ((rc = run_prep(mask, mask_strides, bias, bias_strides, w, want_k, b, h, n, dtype, st))) return rc;

  tri::BwdArgs a;
  a.q = q; a.k = k; a.v = v; a.o = o; a.dout = dout;
  a.packq = w.packq; a.packk = w.packk;
  a.lse = lse;
  a.keep = w.keep; a.rowflag = w.rowflag; a.delta = w.delta; a.lse2 = w.lse2; a.dbpart = w.dbpart;
  a.BH = (int)(b * h);
  a.nchunks = tri::bwd_b_chunks(n, b * h, (int)d * elem_size(dtype));
  a.rows_per_chunk = (int)((n + a.nchunks - 1) / a.nchunks);
  a.dq = dq; a.dk = dk; a.dv = dv; a.db = db;
  a.key_tile0 = 0; a.pass_flags = 0;
  a.dq_lo = w.dbpart;  // (shared with the db partials, which are written after the last pass has read it)
  a.sq = str5(q_strides); a.sk = str5(k_strides); a.sv = str5(v_strides); a.sdo = str5(do_strides);
  a.sdq = str5(dq_strides); a.sdk = str5(dk_strides); a.sdv = str5(dv_strides);
  a.sdb_b = db_strides[0]; a.sdb_h = db_strides[1]; a.sdb_j = db_strides[2]; a.sdb_k = db_strides[3];
  a.H = (int)h; a.N = (int)n; a.NP = w.np; a.nwords = w.nwords;
  a.c = (float)(1.4426950408889634 / std::sqrt((double)d));
  a.sqrt_d = (float)std::sqrt((double)d);
  a.scale = (float)(1.0 / std::sqrt((double)d));
  const int bh = (int)(b * h);
  hipError_t e;
  if (do_q) {
    e = tri::bwd_q_launch(a, bh, (int)d, dtype, tq, st);
    if (e != hipSuccess) return hip_fail(e, "bwd_q launch");
  }
  if (do_kv) {
    e = tri::bwd_kv_launch(a, bh, (int)d, dtype, tkv, st);
    if (e != hipSuccess) return hip_fail(e, "bwd_kv launch");
  }
  if (do_b) {
    e = tri::bwd_b_launch(a, bh, (int)d, dtype, tb, st);
    if (e != hipSuccess) return hip_fail(e, "bwd_b launch");
  }
  return 0;
}

int trifast_bwd(void* dq, void* dk, void* dv, void* db, const void* dout, const void* q, const void* k,
                const void* v, const void* bias, const uint8_t* mask, const void* o, const float* lse,
                int64_t b, int64_t h, int64_t n, int64_t d, int dtype, const int64_t* do_strides,
                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                const int64_t* bias_strides, const int64_t* mask_strides,
                const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                const int64_t* db_strides, const int* tiles,
                void* workspace, int64_t workspace_bytes, void* stream) {
  return bwd_impl(-1, dq, dk, dv, db, dout, q, k, v, bias, mask, o, lse, b, h, n, d, dtype, do_strides,
                  q_strides, k_strides, v_strides, bias_strides, mask_strides, dq_strides, dk_strides,
                  dv_strides, db_strides, tiles, workspace, workspace_bytes, stream);
}

int trifast_bwd_one(int kernel, void* dq, void* dk, void* dv, void* db, const void* dout, const void* q,
                    const void* k, const void* v, const void* bias, const uint8_t* mask, const void* o,
                    const float* lse, int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                    const int64_t* do_strides, const int64_t* q_strides, const int64_t* k_strides,
                    const int64_t* v_strides, const int64_t* bias_strides, const int64_t* mask_strides,
                    const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                    const int64_t* db_strides,
                    int tile, void* workspace, int64_t workspace_bytes, void* stream) {
  if (kernel != TRIFAST_KERNEL_BWD_Q && kernel != TRIFAST_KERNEL_BWD_KV && kernel != TRIFAST_KERNEL_BWD_B)
    return fail(TRIFAST_EINVAL, "kernel id %d is not a backward kernel", kernel);
  int tiles[3] = {-1, -1, -1};
  tiles[kernel - TRIFAST_KERNEL_BWD_Q] = tile;
  return bwd_impl(kernel, dq, dk, dv, db, dout, q, k, v, bias, mask, o, lse, b, h, n, d, dtype, do_strides,
                  q_strides, k_strides, v_strides, bias_strides, mask_strides, dq_strides, dk_strides,
                  dv_strides, db_strides, tiles, workspace, workspace_bytes, stream);
}

namespace {
int gate_impl(bool bwd, void* y_or_dg, void* dox, const void* dy, const void* o, const void* g, int64_t b, int64_t h,
              int64_t n, int64_t d, int dtype, void* stream) {
  g_err[0] = 0;
  if (int rc = check_common(b, h, n, d, dtype)) return rc;
  const void* ptrs[5] = {y_or_dg, o, g, bwd ? dox : o, bwd ? dy : o};
  static const char* const names[5] = {"output", "o", "g", "do", "dy"};
  for (int x = 0; x < 5; ++x) {
    if (!ptrs[x]) return fail(TRIFAST_EINVAL, "gate: %s is a null pointer", names[x]);
    if ((reinterpret_cast<uintptr_t>(ptrs[x]) & 15) != 0) return fail(TRIFAST_EALIGN, "gate: %s is not 16-byte aligned", names[x]);
  }
  tri::GateArgs a;
  a.y = y_or_dg; a.dox = dox; a.o = o; a.g = g; a.dy = dy;
  a.rows = b * n * n; a.plane = n * n; a.H = (int)h; a.D = (int)d;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const hipError_t e = bwd ? tri::gate_launch<true>(a, dtype, st) : tri::gate_launch<false>(a, dtype, st);
  if (e != hipSuccess) return hip_fail(e, "gate launch");
  return 0;
}
}  // namespace

// head dim of a layer whose output is kept heads-outermost (0: plain [rows, n])
static int check_linear_head(const char* what, int p, int64_t n, int64_t hd) {
  if (hd == 0) return 0;
  if (hd < 8 || hd % 8 != 0 || n % hd != 0) return fail(TRIFAST_EINVAL, "%s: layer %d: head dim %lld must be a multiple of 8 that divides its %lld outputs", what, p, (long long)hd, (long long)n);
  return 0;
}

int64_t trifast_linear_dw_workspace_bytes(int64_t rows, int64_t k, int64_t n) {
  if (rows < 1 || k < 1 || n < 1) return fail(TRIFAST_EINVAL, "sizes must be positive");
  return align256(tri::linear_dw_chunks(rows) * n * k * 4) + align256(tri::linear_dw_chunks(rows) * n * 4);
}

int trifast_linear_dw(void* dw, void* db, const void* dy, const void* x, int64_t rows, int64_t k, int64_t n, int64_t head_dim, int dtype,
                      void* workspace, int64_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  if (int rc = check_linear_head("linear_dw", 0, n, head_dim)) return rc;
  if (dtype != TRIFAST_BF16 && dtype != TRIFAST_F16) return fail(TRIFAST_EUNSUPPORTED, "linear_dw: 16-bit element types only (dtype code %d)", dtype);
  if (rows < 1 || n < 1 || n > 65535 * 128) return fail(TRIFAST_EINVAL, "linear_dw: rows and n must be positive (rows=%lld n=%lld)", (long long)rows, (long long)n);
  if (!tri::linear_dw_k_ok(k)) return fail(TRIFAST_EUNSUPPORTED, "linear_dw: %lld input channels (32, 64, 128 or 256 are compiled)", (long long)k);
  if (!dw || !dy || !x) return fail(TRIFAST_EINVAL, "linear_dw: null pointer argument");
  if ((reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(dy) & 15) != 0)
    return fail(TRIFAST_EALIGN, "linear_dw: x and dy must be 16-byte aligned");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0 || workspace_bytes < trifast_linear_dw_workspace_bytes(rows, k, n))
    return fail(TRIFAST_EWORKSPACE, "linear_dw: workspace missing, misaligned or smaller than trifast_linear_dw_workspace_bytes");
  tri::LinearDwArgs a{};
  a.x = x; a.dy = dy; a.dw = dw; a.part = static_cast<float*>(workspace);
  a.db = db;
  a.part_b = db ? reinterpret_cast<float*>(static_cast<char*>(workspace) + align256(tri::linear_dw_chunks(rows) * n * k * 4)) : nullptr;
  a.rows = rows; a.rows_per_chunk = tri::linear_dw_rows_per_chunk(rows); a.chunks = (int)tri::linear_dw_chunks(rows);
  a.K = (int)k; a.N = (int)n; a.hd = (int)head_dim;
  const hipError_t e = tri::linear_dw_launch(a, dtype, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "linear_dw launch");
  return 0;
}

int trifast_linear_fwd(const void* x, int64_t rows, int64_t k, int nlayers, const void* const* w, const void* const* bias,
                       void* const* y, const int64_t* n, const int64_t* head_dim, int dtype, void* stream) {
  g_err[0] = 0;
  if (dtype != TRIFAST_BF16 && dtype != TRIFAST_F16) return fail(TRIFAST_EUNSUPPORTED, "linear_fwd: 16-bit element types only (dtype code %d)", dtype);
  if (rows < 1) return fail(TRIFAST_EINVAL, "linear_fwd: rows must be positive (%lld)", (long long)rows);
  if (!tri::linear_fwd_k_ok(k)) return fail(TRIFAST_EUNSUPPORTED, "linear_fwd: %lld input channels (32, 64 or 128 are compiled)", (long long)k);
  if (nlayers < 1 || nlayers > tri::kLinearLayers) return fail(TRIFAST_EINVAL, "linear_fwd: 1 to %d layers per call (got %d)", tri::kLinearLayers, nlayers);
  if (!x || !w || !y || !n) return fail(TRIFAST_EINVAL, "linear_fwd: null pointer argument");
  if ((reinterpret_cast<uintptr_t>(x) & 15) != 0) return fail(TRIFAST_EALIGN, "linear_fwd: x is not 16-byte aligned");
  tri::LinearFwdArgs a{};
  a.x = x; a.rows = rows; a.K = (int)k; a.nlayers = nlayers;
  for (int p = 0; p < nlayers; ++p) {
    if (!w[p] || !y[p]) return fail(TRIFAST_EINVAL, "linear_fwd: layer %d: null pointer", p);
    if (n[p] < 1 || n[p] > (1 << 20)) return fail(TRIFAST_EINVAL, "linear_fwd: layer %d: %lld outputs", p, (long long)n[p]);
    if ((reinterpret_cast<uintptr_t>(w[p]) & 15) != 0 || (reinterpret_cast<uintptr_t>(y[p]) & 15) != 0)
      return fail(TRIFAST_EALIGN, "linear_fwd: layer %d: weight and output must be 16-byte aligned", p);
    if (int rc = check_linear_head("linear_fwd", p, n[p], head_dim ? head_dim[p] : 0)) return rc;
    a.w[p] = w[p]; a.bias[p] = bias ? bias[p] : nullptr; a.y[p] = y[p]; a.n[p] = (int)n[p]; a.hd[p] = head_dim ? (int)head_dim[p] : 0;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const hipError_t e = dtype == TRIFAST_BF16 ? tri::linear_fwd_launch_t<__bf16>(a, st) : tri::linear_fwd_launch_t<_Float16>(a, st);
  if (e != hipSuccess) return hip_fail(e, "linear_fwd launch");
  return 0;
}

int trifast_linear_dx(void* dx, int64_t rows, int64_t k, int nlayers, const void* const* dy, const void* const* wt,
                      const int64_t* n, const int64_t* head_dim, int dtype, void* stream) {
  g_err[0] = 0;
  if (dtype != TRIFAST_BF16 && dtype != TRIFAST_F16) return fail(TRIFAST_EUNSUPPORTED, "linear_dx: 16-bit element types only (dtype code %d)", dtype);
  if (rows < 1) return fail(TRIFAST_EINVAL, "linear_dx: rows must be positive (%lld)", (long long)rows);
  if (!tri::linear_dx_k_ok(k)) return fail(TRIFAST_EUNSUPPORTED, "linear_dx: %lld input channels (32, 64 or 128 are compiled)", (long long)k);
  if (nlayers < 1 || nlayers > tri::kLinearLayers) return fail(TRIFAST_EINVAL, "linear_dx: 1 to %d layers per call (got %d)", tri::kLinearLayers, nlayers);
  if (!dx || !dy || !wt || !n) return fail(TRIFAST_EINVAL, "linear_dx: null pointer argument");
  if ((reinterpret_cast<uintptr_t>(dx) & 15) != 0) return fail(TRIFAST_EALIGN, "linear_dx: dx is not 16-byte aligned");
  tri::LinearDxArgs a{};
  a.dx = dx; a.rows = rows; a.K = (int)k; a.nlayers = nlayers;
  for (int p = 0; p < nlayers; ++p) {
    if (!dy[p] || !wt[p]) return fail(TRIFAST_EINVAL, "linear_dx: layer %d: null pointer", p);
    if (n[p] < 1 || n[p] > (1 << 20)) return fail(TRIFAST_EINVAL, "linear_dx: layer %d: %lld outputs", p, (long long)n[p]);
    if ((reinterpret_cast<uintptr_t>(dy[p]) & 15) != 0 || (reinterpret_cast<uintptr_t>(wt[p]) & 15) != 0)
      return fail(TRIFAST_EALIGN, "linear_dx: layer %d: dy and the transposed weight must be 16-byte aligned", p);
    if (int rc = check_linear_head("linear_dx", p, n[p], head_dim ? head_dim[p] : 0)) return rc;
    a.dy[p] = dy[p]; a.wt[p] = wt[p]; a.n[p] = (int)n[p]; a.hd[p] = head_dim ? (int)head_dim[p] : 0;
  }
  const hipError_t e = tri::linear_dx_launch(a, dtype, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "linear_dx launch");
  return 0;
}

int trifast_gate_fwd(void* y, const void* o, const void* g, int64_t b, int64_t h, int64_t n, int64_t d, int dtype, void* stream) {
  return gate_impl(false, y, nullptr, nullptr, o, g, b, h, n, d, dtype, stream);
}

int trifast_gate_bwd(void* dout, void* dg, const void* dy, const void* o, const void* g, int64_t b, int64_t h, int64_t n,
                     int64_t d, int dtype, void* stream) {
  return gate_impl(true, dg, dout, dy, o, g, b, h, n, d, dtype, stream);
}

}  // extern "C"
