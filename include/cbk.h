/* cbk.h -- C ABI of the MI355X (gfx950) CBK1 sparse low-bit linear layer.
 *
 * One packed weight matrix W_hat[K, N] (K output rows, N input columns) times fp16/bf16
 * activations X[M, N]:   Y[M, K] = X . W_hat^T (+ bias),  with
 *
 *     W_hat[k, j] = ((q[k, j] - zero[k, j/group]) * scale[k, j/group]) * keep[k, j] * col_scale[cs(k), j]
 *
 * evaluated in float32 (reference: docs/FORMAT.md:43-45, src/cobaltkernel/dequant_ref.py:69-82).
 *
 * Every pointer is a DEVICE pointer owned by the caller.  The library never allocates or
 * frees device memory, never synchronises the host, and launches only on the stream it
 * is given (reference harness: src/cobaltkernel/csrc/test_gemv.cu:187-235 allocates its
 * outputs itself; the runners pre-allocate everything, runner.py:492-521).
 * All entry points return 0 on success or a negative cbk_status.
 */
#ifndef CBK_H_
#define CBK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CBK_ABI_VERSION 1

/* Layout ids 0-7 are the reference's (src/cobaltkernel/csrc/cobalt_format.h:23-32,
 * src/cobaltkernel/pack_cobalt.py:28-36).  8 and 9 generalise the two shipped families to
 * 2/3/4-bit codes, a group of 64 or 128 and any per-32-column survivor count. */
enum cbk_layout {
  CBK_SPARSE4 = 0,   /* bitmap + variable-length nibble stream, per-row offsets          */
  CBK_DENSE4 = 1,    /* 4-bit code per column, pruned columns hold the zero point        */
  CBK_DENSE8 = 2,    /* 8-bit code per column                                            */
  CBK_SPARSE4X = 3,  /* SPARSE4 + uint16 per-group code offsets                          */
  CBK_BF16 = 4,      /* (not supported: unquantised passthrough)                         */
  CBK_SPARSE4E = 5,  /* byte-identical to SPARSE4X                                       */
  CBK_BLK1632_4 = 6, /* exactly 16 of every 32 columns kept, 4-bit survivors             */
  CBK_BLK1632_6 = 7, /* the same mask, 6-bit survivors (nibble plane + hi2 plane)        */
  CBK_BLKC = 8,      /* exactly `keep` of every 32 columns kept, `bits`-bit survivors as
                        one LSB-first bit stream per row; (4,16,128) == BLK1632_4        */
  CBK_DENSEB = 9     /* `bits`-bit code per column as one LSB-first bit stream per row;
                        bits 4 == DENSE4, bits 8 == DENSE8                               */
};

#define CBK_FLAG_ZERO_LE_128 1
#define CBK_FLAG_TILED16 2
#define CBK_FLAG_ZERO_ON_GRID 4

enum cbk_dtype { CBK_F32 = 0, CBK_F16 = 1, CBK_BF16T = 2, CBK_U8 = 3 /* cbk_pack's zero points only */ };

/* gate activations of cbk_linear_act (cobalt_gemm.cuh:216-220: tanh-GELU, x / (1 + exp(-x))) */
enum cbk_act { CBK_ACT_GELU_TANH = 0, CBK_ACT_SILU = 1 };

enum cbk_status {
  CBK_OK = 0,
  CBK_ERR_NULL = -1,        /* a required pointer is NULL                                 */
  CBK_ERR_LAYOUT = -2,      /* unknown layout, or bits/group/keep not valid for it        */
  CBK_ERR_SHAPE = -3,       /* K, N, M, leading dimension or row range out of range       */
  CBK_ERR_ALIGN = -4,       /* a pointer or leading dimension is not aligned as required  */
  CBK_ERR_DTYPE = -5,       /* unsupported element type                                   */
  CBK_ERR_WORKSPACE = -6,   /* workspace missing or smaller than cbk_workspace_bytes()    */
  CBK_ERR_HIP = -7,         /* the HIP runtime reported an error at launch                */
  CBK_ERR_UNSUPPORTED = -8  /* valid descriptor, but this operation does not take it      */
};

/* One packed matrix.  Replaces cbk::Mat (cobalt_format.h:103-109) and the 9-int64 MatDesc
 * device table entry (src/cobaltkernel/csrc/megakernel.cuh:21-28).
 *   data      row regions; fixed-stride layouts: row k at data + k*cbk_row_stride(); 64 B of
 *             readable padding after the last row (docs/FORMAT.md:22-24).  16-byte aligned.
 *   row_off   uint32[K+1] byte offsets of the row regions (SPARSE4/4X/4E only), else NULL
 *   scale     fp16  [K, N/group] row-major, 4-byte aligned
 *   zero      uint8 [K, N/group] row-major integer zero points, 4-byte aligned
 *   col_scale fp16  [cs_rows, N] or NULL (then the factor is 1), 16-byte aligned
 *   cs_rows   1: one vector.  2: fused gate/up, row k uses vector k&1.  3: fused q|k|v, rows
 *             [0,cs_split0) use vector 0, [cs_split0, cs_split0+cs_split1) vector 1, the rest 2
 *             (cobalt_format.h:77-99, docs/FORMAT.md:134-151).  Both kinds run the matrix-core
 *             kernels (q|k|v: decode needs the two boundaries on multiples of 16 rows, prefill
 *             runs range by range unless they are multiples of 256); other splits take the
 *             float row kernel for decode.
 *   bits/group/keep  must be given for layouts 8/9; for 0-7 they may be 0 (implied).
 *   flags     CBK_FLAG_ZERO_LE_128: the caller guarantees that every stored zero point is
 *             <= 128 (always true for an on-grid zero point of a 2/3/4/6-bit code, and for the
 *             reference's off-grid probe, src/cobaltkernel/test_gemv.py:428-431).  The int8
 *             matrix-core decode kernel needs q - zero to fit a signed byte; without the flag
 *             cbk_gemv runs the slower float row kernel, which takes any uint8 zero point.
 *             (The matrix-core kernels take layouts 1, 6, 7, 8, 9 with 2/3/4-bit codes, or 6-bit
 *             for layout 7; SPARSE4X/4E decode on the matrix cores too, 16 rows of different
 *             lengths at a time, SPARSE4, small stream matrices and DENSE8 with integer-dot row
 *             kernels of their own, all of them with the flag only; 8-bit prefill goes through
 *             the generic tile reader.)
 *             CBK_FLAG_TILED16: data / scale / zero are in 16-row tile-interleaved order, a
 *             permutation of the same bytes made once at load time so that the sixteen rows a
 *             wavefront decodes together are contiguous in HBM: with s = cbk_row_stride(),
 *             byte o of row k is at data[(k/16)*16*s + ((o/16)*16 + k%16)*16 + o%16], the
 *             scale / zero entry of (row k, group g) at index ((k/16)*G + g)*16 + k%16; K is
 *             padded with zero rows to a multiple of 16 and data ends with 512 readable bytes.
 *             Fixed-stride layouts only.  Every entry point takes both orders.
 *             CBK_FLAG_ZERO_ON_GRID: the caller guarantees that every stored zero point is
 *             <= 2^bits - 1, i.e. is itself a code.  Only then can a survivor-stream matrix be
 *             re-packed as dense codes (a pruned column of a dense layout stores the zero point
 *             as its code): without the flag cbk_gemm / cbk_linear serve SPARSE4 / 4X / 4E
 *             above 16 rows as 16-row slices on the row kernel, which takes any zero point. */
typedef struct cbk_desc {
  const void* data;
  const void* row_off;
  const void* scale;
  const void* zero;
  const void* col_scale;
  int32_t K, N;
  int32_t layout;
  int32_t bits;
  int32_t group;
  int32_t keep;
  int32_t cs_rows;
  int32_t cs_split0, cs_split1;
  int32_t flags;
} cbk_desc;

int cbk_abi_version(void);
const char* cbk_strerror(int status);

/* Checks a descriptor on the host (no device access) and fills bits/group/keep for the
 * reference layouts into *out (may alias in). */
int cbk_desc_check(const cbk_desc* in, cbk_desc* out);

/* Bytes per row of a fixed-stride layout (cobalt_format.h:59-68); 0 for SPARSE4/4X/4E
 * or an invalid descriptor. */
size_t cbk_row_stride(const cbk_desc* d);

/* Weight bytes one pass over the matrix streams: rows + scale + zero
 * (pack_cobalt.write_matrix :431-433 `stream_bytes`); SPARSE layouts need data_bytes. */
size_t cbk_stream_bytes(const cbk_desc* d, size_t sparse_data_bytes);

/* Device scratch needed by cbk_gemv / cbk_gemm / cbk_linear for M activation rows.  The prefill
 * kernel keeps its pre-scaled fp16 activations there: ceil(M/256)*256 * ceil(N/256)*256 * 2 bytes
 * per col_scale vector, i.e. times cs_rows for a fused matrix, one float32 scale per activation
 * row and col_scale vector, plus float32 partial outputs when the library splits the column range
 * of a launch that would not fill the chip.  The decode kernels need none, with one optional use:
 * two to eight activation rows of rows whose activations take more than 90 KB of LDS
 * (M * 3 * N bytes) are split over the workgroups by columns when there is room for the float32
 * part sums, K * 16 * M * 4 bytes at most, and so are the rows of SPARSE4X / SPARSE4E matrices on
 * the matrix-core stream kernel when the activation rows of a pass (up to eight) do not fit in
 * LDS as whole rows (M * 3 * N bytes beyond about 140 KB); with a smaller workspace, or none,
 * cbk_gemv computes the same bits more slowly and reports no error.
 * Ask, do not compute.  256-byte aligned. */
size_t cbk_workspace_bytes(const cbk_desc* d, int M);

/* Rows [row0, row0+nrows) of W_hat -> out[nrows, ld_out] in out_dtype, bit-exact float32
 * evaluation then one round-to-nearest-even cast.  with_col_scale = 0 leaves the column
 * scale out, like cbk::dequant_row (src/cobaltkernel/csrc/cobalt_gemv.cuh:1218-1315,
 * harness entry `dequant_rows`, test_gemv.cu:223-235). */
int cbk_dequant(const cbk_desc* d, int row0, int nrows, int with_col_scale,
                void* out, int out_dtype, int64_t ld_out, void* stream);

/* RAW arrays -> the data, scale and zero arrays of the CBK1 image `dst` describes (dst->data,
 * dst->scale, dst->zero point at device memory of the sizes the layout implies; CBK_FLAG_TILED16
 * in dst->flags selects the 16-row tiled order, else the reference's row-major order; padding
 * and tail bytes are written as zero).  Fixed-stride layouts only.
 *   mask_bits  uint8 [K, N/8], LSB first, 1 = survivor; NULL = nothing pruned
 *   q          uint8 [K, N] codes (clamped to [0, 2^bits) here)
 *   scale      fp16  [K, N/group]
 *   zero       [K, N/group], zero_dtype CBK_F16 (an integer value, rounded here) or CBK_U8
 * A dense layout stores the group's zero point at a pruned column; a bitmap layout stores the
 * survivors of each 32-column block in column order.  With fix_zero != 0 a group whose zero
 * point lies outside [0, 2^bits - 1] gets scale, zero point and codes re-derived from the hull of
 * its dequantised survivors and 0, as _fix_zero_range does (src/cobaltkernel/pack_cobalt.py:55-87),
 * in correctly rounded float32 steps in that function's order.  `status`, if given, is two device
 * ints the caller has set to 0: bit 0 of status[0] is set when a block does not hold exactly
 * `keep` survivors (the bytes written for such a block are then meaningless), bit 1 when a dense
 * layout had to store, at a pruned column, a zero point above 2^bits - 1 (only its low bits are
 * stored: that column no longer dequantises to 0); status[1] counts the groups re-derived.  The byte layouts are the ones `pack_matrix` (pack_cobalt.py:98-250) writes
 * with torch operations. */
int cbk_pack(const cbk_desc* dst, const void* mask_bits, const void* q, const void* scale,
             const void* zero, int zero_dtype, int fix_zero, int* status, void* stream);

/* The way back: the codes and the keep bitmap of a packed image of any layout, as uint8 [K, N]
 * (0 at a pruned column of a bitmap or survivor-stream layout; a dense layout returns what it
 * stores there, the group's zero point) and, if mask_bits is not NULL, uint8 [K, N/8] LSB first
 * (all ones for a dense layout).  The decode side of `dequant_reference`
 * (src/cobaltkernel/pack_cobalt.py:277-334) without the arithmetic; with cbk_pack it re-packs a
 * matrix into another layout, which is how cbk_gemm serves the survivor-stream layouts. */
int cbk_unpack(const cbk_desc* d, void* q, void* mask_bits, void* stream);

/* Decode path, 1 <= M <= 16: y[m, k] = sum_j x[m, j] * W_hat[k, j] (+ bias[k]).
 * x is [M, ldx] fp16 or bf16, y is [M, ldy] in y_dtype (f32 / f16 / bf16), bias is NULL or
 * K values of y_dtype.  Up to eight activation rows share one pass over the weights on the
 * matrix-core kernel, whatever the row length (two to eight rows of a long row: split over the
 * workgroups by columns through the workspace, see cbk_workspace_bytes, or staged in column slabs
 * without one); more rows, or configurations that kernel takes four rows of at a time, are
 * passes over the weights.  Row m of the result does not depend on M, nor on the workspace.  Replaces the harness
 * entry `gemv` (test_gemv.cu:187-199) and cbk::gemv_rows (cobalt_gemv.cuh:1196-1213); unlike
 * those it applies col_scale itself. */
int cbk_gemv(const cbk_desc* d, const void* x, int x_dtype, int M, int64_t ldx,
             void* y, int y_dtype, int64_t ldy, const void* bias,
             void* workspace, size_t workspace_bytes, void* stream);

/* Several independent decode GEMVs in one kernel launch: the matrices
 * a decoder layer multiplies by the same hidden state (q, k, v; gate, up), or any other set
 * with no data dependence.  n <= 8.  Entry i computes ys[i] = xs[i] . W_hat_i^T (+ biases[i]).
 * Matrices that share (family, bits, group, keep) and qualify for the matrix-core kernel run
 * in one persistent launch that balances their row tiles over the chip; otherwise the call
 * degrades to n single calls.  workspace >= cbk_gemv_batch_workspace_bytes(), 256-byte aligned.
 * Counterpart of the reference's fused row-concatenated matrices (docs/FORMAT.md:126-151) and
 * of the harness entry `gemv_multi` (src/cobaltkernel/csrc/test_gemv.cu:237-291). */
size_t cbk_gemv_batch_workspace_bytes(int n, const cbk_desc* descs, int M);
int cbk_gemv_batch(int n, const cbk_desc* descs, const void* const* xs, const int64_t* ldxs,
                   int x_dtype, int M, void* const* ys, const int64_t* ldys, int y_dtype,
                   const void* const* biases, void* workspace, size_t workspace_bytes, void* stream);

/* Prefill path, any M >= 1 (256-token tiles; a 128-token tile up to 128 rows, a 64-token tile up to 64).  Same contract as
 * cbk_gemv; activations are carried as fp16 inside, a token whose values leave fp16's range
 * scaled by a power of two on the way in and back on the way out.  The survivor-stream layouts
 * (SPARSE4, SPARSE4X, SPARSE4E) are re-packed for the call, above 16 rows, into the dense 4-bit
 * layout inside the workspace (cbk_workspace_bytes counts it) when the descriptor carries
 * CBK_FLAG_ZERO_ON_GRID, has at most one col_scale vector and the workspace is large enough;
 * otherwise, and up to 16 rows, they go to the row kernel in slices of 16 activation rows,
 * which needs no workspace.  Replaces the harness entry `gemm` (test_gemm.cu:151-165) and cbk::gemm_tile
 * (cobalt_gemm.cuh:243-609). */
int cbk_gemm(const cbk_desc* d, const void* x, int x_dtype, int M, int64_t ldx,
             void* y, int y_dtype, int64_t ldy, const void* bias,
             void* workspace, size_t workspace_bytes, void* stream);

/* cbk_gemm for callers that cannot allocate device memory or pass a workspace: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same computation and same results as cbk_gemm, with the scratch (pre-scaled
 * activations, partial output tiles) in an array of CBK_STATIC_SCRATCH_BYTES that is part of the
 * library's device image: every GPU the library runs on holds one copy until the process ends.
 * The call allocates and frees nothing.  A call whose cbk_workspace_bytes() exceeds the array is
 * refused with CBK_ERR_WORKSPACE before anything is launched (16 MiB hold e.g. 1024 activation
 * rows of 5376 columns; prompts beyond that go through cbk_gemm).  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race;
 * calls on one stream are safe.  Nothing in the array needs to start at zero and nothing is
 * carried from one call to the next.  The first call on a GPU looks up the array's address
 * there, and the first call of each kernel configuration sets a kernel attribute: neither can
 * be recorded, so make one call per GPU and configuration (same layout, code width, row count
 * class) outside stream capture before capturing calls of it into a graph. */
#define CBK_STATIC_SCRATCH_BYTES (16u << 20)
int cbk_gemm_static(const cbk_desc* d, const void* x, int x_dtype, int M, int64_t ldx,
                    void* y, int y_dtype, int64_t ldy, const void* bias, void* stream);

/* The layer forward: cbk_gemv for M <= 8, cbk_gemm above (the module seam of
 * benchmarks/benchmark_suite.py:1200-1217). */
int cbk_linear(const cbk_desc* d, const void* x, int x_dtype, int M, int64_t ldx,
               void* y, int y_dtype, int64_t ldy, const void* bias,
               void* workspace, size_t workspace_bytes, void* stream);

/* The first half of a gated MLP in one call, for a matrix whose rows 2i / 2i+1 are the gate and
 * up rows of output i (K even; normally cs_rows == 2):
 *   y[m, i] = act(t[m, 2i]) * t[m, 2i+1],   t = x . W_hat^T (+ bias, K entries of type y_dtype),
 * y [M, K/2] with ldy >= K/2.  Up to 128 activation rows t is kept in float32 and the result is
 * rounded once, as EPI_GEGLU_BF16 / EPI_SWIGLU_BF16 of cbk::gemm_tile do
 * (cobalt_gemm.cuh:30-33, :586-592; checked by test_gemm.py:196-210); above that t is stored in
 * y_dtype between the matrix kernel and the activation kernel (one more rounding of gate and
 * up).  The workspace holds t and the scratch of cbk_linear: cbk_linear_act_workspace_bytes(). */
size_t cbk_linear_act_workspace_bytes(const cbk_desc* d, int M, int y_dtype);
int cbk_linear_act(const cbk_desc* d, const void* x, int x_dtype, int M, int64_t ldx,
                   void* y, int y_dtype, int64_t ldy, const void* bias, int act,
                   void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CBK_H_ */
