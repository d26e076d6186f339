/*
 * trifast_hip.h -- C ABI of the MI355X (gfx950) triangle self-attention kernels.
 *
 * This is the boundary that replaces the host->device launches of the reference
 * operator (reference src/trifast/torch.py:48-59 for forward, :111-174 for the
 * three backward launches): raw device pointers, element strides, sizes, a dtype
 * code, a tile id and a HIP stream.  No torch types cross it.
 *
 * Conventions
 *   - Every entry point returns 0 on success, a negative TRIFAST_E* code for a
 *     rejected argument, or a positive hipError_t for a failed launch.  The text
 *     of the last failure on the calling thread is in trifast_last_error().
 *   - Tensors are owned by the caller.  The library never allocates or frees
 *     device memory and keeps no pointer after a call returns; temporary storage
 *     is a caller-provided workspace whose size trifast_*_workspace_bytes gives.
 *   - Launches are asynchronous on `stream` (a hipStream_t passed as void*).
 *   - Layouts (reference src/trifast/torch.py:220-226):
 *       q, k, v, do : [b, h, n, n, d]  element strides {sb, sh, si, sj, sd}, sd == 1
 *       bias        : [b, h, n, n]     element strides {sb, sh, sj, sk}, any
 *       mask        : [b, n, n] bytes  strides {sb, si, sk}, any; nonzero = key masked OUT
 *       o           : contiguous [b, h, n, n, d]
 *       dq, dk, dv  : [b, h, n, n, d]  element strides like q (sd == 1), or contiguous
 *       db          : [b, h, n, n]     element strides {sb, sh, sj, sk}, any, or contiguous
 *       lse         : contiguous float32 [b, h, n, n], natural log, indexed [i, j]
 *     Vector accesses need 16-byte alignment: base pointers of q, k, v, do, o, dq, dk,
 *     dv, db must be 16-byte aligned and the si/sj/sh/sb strides of the q-like ones
 *     multiples of 16/sizeof(elem), with 0 <= sj * sizeof(elem) < 2^24 (the rows of a tile
 *     are addressed with 32-bit offsets); lse must be 4-byte aligned.  Outputs must not
 *     overlap themselves or each other (no zero strides over a dim larger than 1).
 *     bias and mask are re-tiled by pre-pass kernels into the workspace, so they
 *     carry no alignment or contiguity requirement.
 */
#ifndef TRIFAST_HIP_H
#define TRIFAST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRIFAST_ABI_VERSION 3

/* dtype codes */
#define TRIFAST_F32 0
#define TRIFAST_BF16 1
#define TRIFAST_F16 2

/* kernel ids: one per launch of the reference operator
 * (reference src/trifast/triton.py:19 _fwd, :274 _bwd_q, :143 _bwd_kv, :394 _bwd_b) */
#define TRIFAST_KERNEL_FWD 0
#define TRIFAST_KERNEL_BWD_Q 1
#define TRIFAST_KERNEL_BWD_KV 2
#define TRIFAST_KERNEL_BWD_B 3
#define TRIFAST_NUM_KERNELS 4

/* error codes */
#define TRIFAST_OK 0
#define TRIFAST_EINVAL (-1)      /* bad size / null pointer / bad dtype            */
#define TRIFAST_EUNSUPPORTED (-2) /* head dim or tile not among the compiled ones */
#define TRIFAST_EALIGN (-3)      /* pointer or stride breaks the alignment rule    */
#define TRIFAST_EWORKSPACE (-4)  /* workspace missing or too small                 */

int trifast_abi_version(void);

/* Text of the last error on this thread ("" if none). */
const char* trifast_last_error(void);

/*
 * Maximum shader clock of a device in MHz (negative error code on failure).  No
 * counterpart in the reference: the benchmark uses it to state the matrix peak at the
 * device's own clock next to the nominal one.
 */
int trifast_device_clock_mhz(int device);

/*
 * Compiled tile instantiations, for the tuner.  Replaces the triton.Config lists
 * of reference src/trifast/autotune_helpers.py:58-211.
 *   trifast_num_tiles(kernel)            number of instantiations of that kernel
 *   trifast_tile_info(kernel, tile, ...) block sizes of one instantiation
 *   trifast_supports(...)                1 if the instantiation can run the shape
 *   trifast_default_tile(...)            heuristic pick when nothing is cached
 */
int trifast_num_tiles(int kernel);
int trifast_tile_info(int kernel, int tile, int* block_j, int* block_k, int* num_waves);
int trifast_supports(int kernel, int tile, int64_t n, int64_t h, int64_t d, int dtype);
int trifast_default_tile(int kernel, int64_t n, int64_t h, int64_t d, int dtype);

/*
 * 1 for the tiles of TRIFAST_KERNEL_BWD_KV that keep a whole pair row in one
 * workgroup and produce dq, dk and dv from one computation of the scores (the
 * reference runs _bwd_q and _bwd_kv for this, src/trifast/torch.py:111-149): with such
 * a tile trifast_bwd does not launch the dq kernel, and trifast_bwd_one(BWD_KV) writes
 * dq as well.  0 for every other tile.
 */
int trifast_bwd_kv_tile_writes_dq(int tile);

/* Bytes of caller-provided workspace (256-byte aligned) each call needs: O(b h n^2); the
 * backward's is b h n^2 (12 + 4 chunks) bytes for 16-bit inputs (chunks of pair rows of the
 * bias gradient, at most 8) or, for rows of 1025..8192 keys at head dim 32, b h n^2 (12 + 2 d)
 * (the row-resident kernel then keeps dq between its passes over the keys as two 16-bit
 * numbers per value, the second of them in the workspace). */
int64_t trifast_fwd_workspace_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int dtype);
int64_t trifast_bwd_workspace_bytes(int64_t b, int64_t h, int64_t n, int64_t d, int dtype);

/*
 * Forward: o, lse = triangle_attention(q, k, v, bias, mask).
 * Replaces the _fwd launch of reference src/trifast/torch.py:48-59.
 * tile < 0 selects trifast_default_tile.
 */
int trifast_fwd(void* o, float* lse,
                const void* q, const void* k, const void* v,
                const void* bias, const uint8_t* mask,
                int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                const int64_t* bias_strides, const int64_t* mask_strides,
                int tile, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Forward without a workspace argument and without any allocation.  No counterpart
 * in the reference: it is for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * Same arguments and results as trifast_fwd; the keep words, row flags and packed
 * bias tiles live in a static device array of TRIFAST_STATIC_SCRATCH_BYTES inside
 * the library (one copy per GPU, held until the process ends).  A shape whose
 * trifast_fwd_workspace_bytes exceeds that is rejected with TRIFAST_EWORKSPACE
 * (bf16/fp16: b*h*ceil(n/32)^2 <= 6100 or so, e.g. b=1 h=4 n=1024).  The pre-passes
 * rewrite every byte the kernel reads, so nothing has to be cleared between calls.
 * All calls on one GPU share the array: calls that overlap on one GPU (different
 * streams or threads) race; serialise them on one stream.
 */
#define TRIFAST_STATIC_SCRATCH_BYTES (12 * 1024 * 1024)
int trifast_fwd_static(void* o, float* lse,
                       const void* q, const void* k, const void* v,
                       const void* bias, const uint8_t* mask,
                       int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                       const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                       const int64_t* bias_strides, const int64_t* mask_strides,
                       int tile, void* stream);

/*
 * Backward: dq, dk, dv, db from do and the saved q, k, v, bias, mask, o, lse.
 * Replaces the _bwd_q, _bwd_kv and _bwd_b launches of reference
 * src/trifast/torch.py:111-174 (one call, fixed launch order, deterministic).
 * do may have any strides over b, h, i, j (stride 0 included, as a broadcast
 * gradient has), but its rows must be 16-byte aligned with last stride 1: the
 * caller materialises a do that is not.  o and lse are the forward's contiguous
 * outputs.  tiles[3] = {bwd_q, bwd_kv, bwd_b} tile ids (<0: default).
 * dq/dk/dv/db_strides give the layout the gradients are written in (NULL:
 * contiguous).  The reference's backward allocates its gradients like its saved,
 * possibly strided inputs (src/trifast/torch.py:85-104); passing the inputs' own
 * strides lets a caller hand the gradients to leaves that are transposed views
 * without a re-layout copy.
 */
int trifast_bwd(void* dq, void* dk, void* dv, void* db,
                const void* dout, const void* q, const void* k, const void* v,
                const void* bias, const uint8_t* mask, const void* o, const float* lse,
                int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                const int64_t* do_strides, const int64_t* q_strides, const int64_t* k_strides,
                const int64_t* v_strides, const int64_t* bias_strides, const int64_t* mask_strides,
                const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                const int64_t* db_strides,
                const int* tiles, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * The three backward launches one at a time (same arguments as trifast_bwd; each
 * writes only its own outputs), so a tuner can time them separately.  Order
 * matters exactly as in the reference (src/trifast/torch.py:110): BWD_Q first --
 * it also fills the workspace's delta = rowsum(o * do) that the other two read.
 * A BWD_KV tile for which trifast_bwd_kv_tile_writes_dq is 1 needs no BWD_Q before
 * it: it writes dq and fills the workspace itself.
 */
int trifast_bwd_one(int kernel,
                    void* dq, void* dk, void* dv, void* db,
                    const void* dout, const void* q, const void* k, const void* v,
                    const void* bias, const uint8_t* mask, const void* o, const float* lse,
                    int64_t b, int64_t h, int64_t n, int64_t d, int dtype,
                    const int64_t* do_strides, const int64_t* q_strides, const int64_t* k_strides,
                    const int64_t* v_strides, const int64_t* bias_strides, const int64_t* mask_strides,
                    const int64_t* dq_strides, const int64_t* dk_strides, const int64_t* dv_strides,
                    const int64_t* db_strides,
                    int tile, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Weight gradient of a linear layer over a pair representation: dw[n, k] = sum over r of
 * dy[r, n] x[r, k] for x [rows, k], dy [rows, n], dw [n, k], all dense, of one 16-bit dtype,
 * rows = b n^2 in the millions and k in {32, 64, 128, 256}: the rows are split over
 * workgroups, whose fp32 partials (the workspace) are added in a fixed order.  db, if not null,
 * receives the layer's bias gradient db[n] = sum over r of dy[r, n] from the same pass.  head_dim = 0:
 * dy is [rows, n]; head_dim = d: dy is kept heads-outermost, [n / d][rows][d], the layout the
 * attention operator takes q, k, v in (d a multiple of 8 that divides n).  No counterpart
 * in the reference, whose callers are only hinted at by the module of
 * tests/unit/test_trifast.py:152-169 (its q, k, v, bias linear layers, trained in :172-210).
 */
int64_t trifast_linear_dw_workspace_bytes(int64_t rows, int64_t k, int64_t n);
/*
 * Up to 6 linear layers over the same pair representation in one pass that reads x once:
 * y_p = x W_p^T + bias_p for x [rows, k], W_p [n_p, k], bias_p [n_p] or null, y_p [rows, n_p]
 * (all dense, one 16-bit dtype, k in {32, 64, 128}).  w, bias, y, n are host arrays of nlayers
 * entries (bias itself may be null: no layer has one; head_dim may be null: every y_p is
 * [rows, n_p]; head_dim[p] = d writes y_p heads-outermost, see trifast_linear_dw).  No counterpart
 * in the reference (see trifast_linear_dw).
 */
int trifast_linear_fwd(const void* x, int64_t rows, int64_t k, int nlayers, const void* const* w, const void* const* bias,
                       void* const* y, const int64_t* n, const int64_t* head_dim, int dtype, void* stream);
/*
 * Input gradient of up to 6 linear layers over the same pair representation in one pass:
 * dx[r, :] = sum over layers p of dy_p[r, :] W_p, with dy_p [rows, n_p] and the weights given
 * transposed, wt_p = W_p^T [k, n_p] (all dense, one 16-bit dtype, k in {32, 64, 128}); every
 * dy_p is read once and dx [rows, k] written once.  dy, wt, n, head_dim are host arrays of
 * nlayers entries (head_dim may be null; see trifast_linear_dw).  No counterpart in the reference (see trifast_linear_dw).
 */
int trifast_linear_dx(void* dx, int64_t rows, int64_t k, int nlayers, const void* const* dy, const void* const* wt,
                      const int64_t* n, const int64_t* head_dim, int dtype, void* stream);
int trifast_linear_dw(void* dw, void* db, const void* dy, const void* x, int64_t rows, int64_t k, int64_t n, int64_t head_dim, int dtype,
                      void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Output gating of a triangle-attention block, fused with the layout change between the
 * operator and the block's output projection.  No counterpart in the reference (its callers
 * are only hinted at by the module of reference tests/unit/test_trifast.py:152-169): this is
 * the caller-side step that follows trifast_fwd in an AlphaFold-style block.
 *   forward   y[b, i, j, h, :]  = o[b, h, i, j, :] * sigmoid(g[b, i, j, h, :])
 *   backward  do[b, h, i, j, :] = dy[b, i, j, h, :] * sigmoid(g)
 *             dg[b, i, j, h, :] = dy * o * sigmoid(g) * (1 - sigmoid(g))
 * o, do: the operator's layout [b, h, n, n, d]; g, dg, y, dy: [b, n, n, h, d], the layout of a
 * linear layer over the pair representation.  All tensors contiguous, 16-byte aligned, of
 * dtype `dtype`; arithmetic in fp32.  Nothing is allocated; the launch is asynchronous on
 * `stream`.
 */
int trifast_gate_fwd(void* y, const void* o, const void* g,
                     int64_t b, int64_t h, int64_t n, int64_t d, int dtype, void* stream);
int trifast_gate_bwd(void* dout, void* dg, const void* dy, const void* o, const void* g,
                     int64_t b, int64_t h, int64_t n, int64_t d, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRIFAST_HIP_H */
