// extern "C" surface of libcbk_hip.so: host-side descriptor checks and kernel dispatch.
// No allocation, no host synchronisation; the only global state is the scratch array of
// cbk_gemm_static and its per-device address.
#include <mutex>
#include "cbk_device.h"

namespace cbk {
int launch_dequant(const DMat&, int, int, int, void*, int, int64_t, hipStream_t);
int launch_gemv_generic(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*, void*, size_t,
                        hipStream_t);
size_t gemv_stream_workspace(const DMat&, int M);
struct GvCall { DMat m; const void* x; int64_t ldx; void* y; int64_t ldy; const void* bias; int par; };
int launch_gemv_fast_batch(int n, const GvCall* calls, int xdt, int M, int ydt, void* ws, size_t ws_bytes,
                           hipStream_t);
bool gemv_fast_takes(const DMat&, int M);
bool gemv_same_config(const DMat&, const DMat&);
size_t gemv_fast_workspace(const DMat&, int M);
constexpr int kMaxBatch = 8;
int launch_act_mul(const void* t, int tdt, int64_t ldt, void* y, int ydt, int64_t ldy, int M, int K2, int act,
                   const void* bias, hipStream_t st, bool halves = false);
int launch_gemm(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*,
                hipStream_t);
int launch_gemm_big(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*, void*, size_t,
                    hipStream_t, bool halves = false);
size_t gemm_big_workspace(const DMat&, int M);
int launch_pack(const DMat&, const void* mask, const void* q, const void* scale, const void* zero, int zero_f16,
                int fix_zero, int* status, hipStream_t);
int launch_unpack(const DMat&, void* q, void* mask, hipStream_t);
// The 256 x 256 tile kernel takes every call of the fixed-stride layouts: below 256 activation
// rows part of its token tile is padding, and it is still several times faster than the
// 128 x 128 kernel, which decodes through the generic reader (14336 x 4096 at 64 rows: 54 us
// against 288 us).  That one stays for q|k|v matrices whose ranges are off the 16-row grid.
static inline bool gemm_big_takes(const DMat& m, int M) {
  if (M < 1 || family_of(m.layout) == FAM_SPARSE) return false;
  return m.cs_rows <= 2 || (m.cs_split0 % 256 == 0 && (m.cs_split0 + m.cs_split1) % 256 == 0);
}

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Row range [lo, hi) of a fixed-stride matrix as a matrix of its own with a single col_scale
// vector (row `cs_row` of the fused one).  lo is a multiple of 16, so the range is a contiguous
// byte slice of data, scale and zero in the row-major and in the tiled order alike.
static DMat row_range(const DMat& m, int lo, int hi, int cs_row) {
  DMat s = m;
  s.data = m.data + (size_t)lo * m.stride;
  s.scale = m.scale + (size_t)lo * m.G;
  s.zero = m.zero + (size_t)lo * m.G;
  s.K = hi - lo;
  s.cs = m.cs ? m.cs + (size_t)cs_row * m.N : nullptr;
  s.cs_rows = m.cs ? 1 : 0;
  s.cs_split0 = s.cs_split1 = 0;
  return s;
}

// The q|k|v ranges of a matrix with three col_scale vectors, if each starts on a 16-row tile.
// Returns the number of non-empty ranges (0: not decomposable).
static int fused_ranges(const DMat& m, int (&lo)[3], int (&hi)[3], int (&row)[3]) {
  if (m.cs_rows != 3 || family_of(m.layout) == FAM_SPARSE) return 0;
  const int b0 = m.cs_split0, b1 = m.cs_split0 + m.cs_split1;
  if (b0 % 16 || b1 % 16) return 0;
  const int l[3] = {0, b0, b1}, h[3] = {b0, b1, m.K};
  int n = 0;
  for (int r = 0; r < 3; ++r)
    if (h[r] > l[r]) { lo[n] = l[r]; hi[n] = h[r]; row[n] = r; ++n; }
  return n;
}

// One call of the decode kernel per col_scale vector: a q|k|v matrix becomes up to three row
// ranges; a gate/up matrix (two vectors by row parity) stays whole and is marked `par`, the
// kernel then stages both scaled activation vectors and every row keeps the sum of its own.
static int expand_fused(const GvCall& c, size_t ysz, GvCall* out) {
  if (c.m.cs_rows != 3) {
    out[0] = c;
    out[0].par = c.m.cs_rows == 2 ? 1 : 0;
    return 1;
  }
  int lo[3], hi[3], row[3];
  const int n = fused_ranges(c.m, lo, hi, row);
  for (int i = 0; i < n; ++i) {
    out[i] = c;
    out[i].m = row_range(c.m, lo[i], hi[i], row[i]);
    out[i].y = (uint8_t*)c.y + (size_t)lo[i] * ysz;
    out[i].bias = c.bias ? (const uint8_t*)c.bias + (size_t)lo[i] * ysz : nullptr;
    out[i].par = 0;
  }
  return n;
}

static int canon(const cbk_desc* in, cbk_desc* o) {
  if (!in || !o) return CBK_ERR_NULL;
  cbk_desc d = *in;
  switch (d.layout) {
    case CBK_DENSE4: d.bits = 4; d.group = 128; d.keep = 0; break;
    case CBK_DENSE8: d.bits = 8; d.group = 128; d.keep = 0; break;
    case CBK_SPARSE4: case CBK_SPARSE4X: case CBK_SPARSE4E: d.bits = 4; d.group = 128; d.keep = 0; break;
    case CBK_BLK1632_4: d.bits = 4; d.group = 128; d.keep = 16; break;
    case CBK_BLK1632_6: d.bits = 6; d.group = 128; d.keep = 16; break;
    case CBK_BLKC:
      if (!(d.bits == 2 || d.bits == 3 || d.bits == 4)) return CBK_ERR_LAYOUT;
      if (d.keep < 1 || d.keep > 32) return CBK_ERR_LAYOUT;
      break;
    case CBK_DENSEB:
      if (!(d.bits == 2 || d.bits == 3 || d.bits == 4 || d.bits == 8)) return CBK_ERR_LAYOUT;
      d.keep = 0;
      break;
    default: return CBK_ERR_LAYOUT;
  }
  if (d.group != 64 && d.group != 128) return CBK_ERR_LAYOUT;
  if (d.K <= 0 || d.N <= 0 || d.N % 128 != 0) return CBK_ERR_SHAPE;
  if (d.cs_rows < 0 || d.cs_rows > 3) return CBK_ERR_SHAPE;
  if (d.cs_rows == 3 && (d.cs_split0 < 0 || d.cs_split1 < 0 || d.cs_split0 + d.cs_split1 > d.K))
    return CBK_ERR_SHAPE;
  *o = d;
  return CBK_OK;
}

static size_t stride_of(const cbk_desc& d) {
  switch (family_of(d.layout)) {
    case FAM_DENSE: return align_up(((size_t)d.N * d.bits + 7) / 8, 16);
    case FAM_BLK: return (size_t)d.N / 8 + align_up(((size_t)(d.N / 32) * d.keep * d.bits + 7) / 8, 16);
    case FAM_BLK6: return (size_t)d.N / 2;
    default: return 0;
  }
}

static int to_dmat(const cbk_desc* in, DMat* m, bool need_device_ptrs) {
  cbk_desc d;
  int rc = canon(in, &d);
  if (rc) return rc;
  const bool sparse = family_of(d.layout) == FAM_SPARSE;
  if (need_device_ptrs) {
    if (!d.data || !d.scale || !d.zero) return CBK_ERR_NULL;
    if (sparse && !d.row_off) return CBK_ERR_NULL;
    if (d.cs_rows > 0 && !d.col_scale) return CBK_ERR_NULL;
    if (((uintptr_t)d.data & 15) || ((uintptr_t)d.scale & 3) || ((uintptr_t)d.zero & 3) ||
        ((uintptr_t)d.col_scale & 15) || ((uintptr_t)d.row_off & 3))
      return CBK_ERR_ALIGN;
  }
  m->data = (const uint8_t*)d.data;
  m->row_off = (const uint32_t*)d.row_off;
  m->scale = (const uint16_t*)d.scale;
  m->zero = (const uint8_t*)d.zero;
  m->cs = d.cs_rows > 0 ? (const uint16_t*)d.col_scale : nullptr;
  m->K = d.K; m->N = d.N; m->G = d.N / d.group;
  m->layout = d.layout; m->bits = d.bits; m->group = d.group; m->keep = d.keep;
  m->cs_rows = d.cs_rows; m->cs_split0 = d.cs_split0; m->cs_split1 = d.cs_split1;
  m->flags = d.flags;
  m->tiled = (d.flags & CBK_FLAG_TILED16) ? 1 : 0;
  if (m->tiled && sparse) return CBK_ERR_UNSUPPORTED;
  m->stride = (uint32_t)stride_of(d);
  m->code_off = family_of(d.layout) == FAM_DENSE ? 0u : (uint32_t)(d.N / 8);
  return CBK_OK;
}

static int check_io(const void* x, int xdt, int M, int64_t ldx, const void* y, int ydt, int64_t ldy, int N,
                    int K) {
  if (!x || !y) return CBK_ERR_NULL;
  if (xdt != CBK_F16 && xdt != CBK_BF16T) return CBK_ERR_DTYPE;
  if (ydt != CBK_F32 && ydt != CBK_F16 && ydt != CBK_BF16T) return CBK_ERR_DTYPE;
  if (M < 1 || ldx < N || ldy < K) return CBK_ERR_SHAPE;
  if (((uintptr_t)x & 15) || (ldx & 7)) return CBK_ERR_ALIGN;
  if ((uintptr_t)y & (ydt == CBK_F32 ? 3 : 1)) return CBK_ERR_ALIGN;
  return CBK_OK;
}

// A survivor-stream matrix (SPARSE4, SPARSE4X, SPARSE4E: rows of different lengths) has no
// matrix-core kernel of its own.  A prefill call re-packs it, in the caller's workspace and for
// the duration of the call, as the dense 4-bit layout in tiled order (pruned columns hold the
// zero point, so every weight dequantises to the same value) and runs the prefill kernel on that:
// two small kernels (image -> codes and bitmap, codes -> rows) in front of the matrix product.
// A pruned column of the dense image stores the zero point as its code, so this needs every zero
// point to be a 4-bit code itself (CBK_FLAG_ZERO_ON_GRID: the host cannot look), and a fixed row
// stride cannot carry row-fused column scales; such matrices, and calls without the workspace,
// are served by the row kernel in slices of 16 activation rows.
static inline bool sparse_repackable(const DMat& m) {
  return m.cs_rows <= 1 && (m.flags & CBK_FLAG_ZERO_ON_GRID) != 0;
}
struct Transient {
  size_t q, mask, data, scale, zero, end;   // byte offsets in the workspace, 256-byte aligned
};
static Transient transient_dense4(const DMat& m) {
  const size_t K16 = ((size_t)m.K + 15) / 16 * 16, stride = (size_t)m.N / 2;
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  Transient t;
  t.q = 0;
  t.mask = up((size_t)m.K * m.N);
  t.data = t.mask + up((size_t)m.K * (m.N / 8));
  t.scale = t.data + up(K16 * stride + 512);
  t.zero = t.scale + up(K16 * m.G * 2);
  t.end = t.zero + up(K16 * m.G);
  return t;
}
static DMat dense4_view(const DMat& m, uint8_t* ws, const Transient& t) {
  DMat d = m;
  d.row_off = nullptr;
  if (ws) { d.data = ws + t.data; d.scale = (const uint16_t*)(ws + t.scale); d.zero = ws + t.zero; }   // else: sizes only
  d.layout = CBK_DENSE4; d.bits = 4; d.group = 128; d.keep = 0; d.G = m.N / 128;
  d.flags = m.flags | CBK_FLAG_TILED16;                             // CBK_FLAG_ZERO_LE_128 as the caller stated it
  d.tiled = 1;
  d.stride = (uint32_t)(m.N / 2); d.code_off = 0;
  return d;
}

}  // namespace cbk

using namespace cbk;

extern "C" {

int cbk_abi_version(void) { return CBK_ABI_VERSION; }

const char* cbk_strerror(int s) {
  switch (s) {
    case CBK_OK: return "ok";
    case CBK_ERR_NULL: return "a required pointer is NULL";
    case CBK_ERR_LAYOUT: return "unknown layout or invalid bits/group/keep for it";
    case CBK_ERR_SHAPE: return "shape, leading dimension or row range out of range";
    case CBK_ERR_ALIGN: return "pointer or leading dimension not aligned as required";
    case CBK_ERR_DTYPE: return "unsupported element type";
    case CBK_ERR_WORKSPACE: return "workspace missing or too small";
    case CBK_ERR_HIP: return "HIP runtime error at launch";
    case CBK_ERR_UNSUPPORTED: return "operation does not support this layout";
    default: return "unknown status";
  }
}

int cbk_desc_check(const cbk_desc* in, cbk_desc* out) { return canon(in, out); }

size_t cbk_row_stride(const cbk_desc* in) {
  cbk_desc d;
  if (canon(in, &d)) return 0;
  return stride_of(d);
}

size_t cbk_stream_bytes(const cbk_desc* in, size_t sparse_data_bytes) {
  cbk_desc d;
  if (canon(in, &d)) return 0;
  const size_t meta = (size_t)d.K * (d.N / d.group) * 3;
  if (family_of(d.layout) == FAM_SPARSE) return sparse_data_bytes + meta;
  return (size_t)d.K * stride_of(d) + meta;
}

size_t cbk_workspace_bytes(const cbk_desc* in, int M) {
  DMat m;
  if (to_dmat(in, &m, false)) return 0;
  if (family_of(m.layout) == FAM_SPARSE) {                          // cbk_gemm / cbk_linear above 16 rows: see Transient
    if (M <= 16) return gemv_stream_workspace(m, M);                // part sums of long rows split by columns, else none
    if (!sparse_repackable(m)) return 0;
    const Transient t = transient_dense4(m);
    return t.end + gemm_big_workspace(dense4_view(m, nullptr, t), M);
  }
  // the most any of the three entry points asks for (cbk_gemm runs the prefill kernel at any M)
  size_t need = (M >= 1 && M <= 16 && gemv_fast_takes(m, 1)) ? gemv_fast_workspace(m, M) : 0;
  if (gemm_big_takes(m, M)) {
    const size_t b = gemm_big_workspace(m, M);
    return need > b ? need : b;
  }
  int lo[3], hi[3], row[3];
  const int nr = M >= 1 ? fused_ranges(m, lo, hi, row) : 0;
  for (int i = 0; i < nr; ++i) {                                    // run one after the other on the same bytes
    const size_t b = gemm_big_workspace(row_range(m, lo[i], hi[i], row[i]), M);
    need = need > b ? need : b;
  }
  return need;
}

size_t cbk_gemv_batch_workspace_bytes(int n, const cbk_desc* descs, int M) {
  size_t total = 0;
  for (int i = 0; i < n; ++i) total += cbk_workspace_bytes(descs + i, M);
  return total;
}

int cbk_dequant(const cbk_desc* in, int row0, int nrows, int with_col_scale, void* out, int out_dtype,
                int64_t ld_out, void* stream) {
  DMat m;
  int rc = to_dmat(in, &m, true);
  if (rc) return rc;
  if (!out) return CBK_ERR_NULL;
  if (row0 < 0 || nrows < 0 || row0 + nrows > m.K || ld_out < m.N) return CBK_ERR_SHAPE;
  if (out_dtype != CBK_F32 && out_dtype != CBK_F16 && out_dtype != CBK_BF16T) return CBK_ERR_DTYPE;
  return launch_dequant(m, row0, nrows, with_col_scale, out, out_dtype, ld_out, (hipStream_t)stream);
}

int cbk_pack(const cbk_desc* dst, const void* mask_bits, const void* q, const void* scale, const void* zero,
             int zero_dtype, int fix_zero, int* status, void* stream) {
  DMat m;
  const int rc = to_dmat(dst, &m, true);
  if (rc) return rc;
  if (!q || !scale || !zero) return CBK_ERR_NULL;
  if (zero_dtype != CBK_F16 && zero_dtype != CBK_U8) return CBK_ERR_DTYPE;
  if (((uintptr_t)q & 15) || ((uintptr_t)mask_bits & 3) || ((uintptr_t)scale & 1) || ((uintptr_t)status & 3) ||
      (zero_dtype == CBK_F16 && ((uintptr_t)zero & 1)))
    return CBK_ERR_ALIGN;
  return launch_pack(m, mask_bits, q, scale, zero, zero_dtype == CBK_F16, fix_zero != 0, status, (hipStream_t)stream);
}

int cbk_unpack(const cbk_desc* in, void* q, void* mask_bits, void* stream) {
  DMat m;
  const int rc = to_dmat(in, &m, true);
  if (rc) return rc;
  if (!q) return CBK_ERR_NULL;
  if (((uintptr_t)q & 15) || ((uintptr_t)mask_bits & 3)) return CBK_ERR_ALIGN;
  return launch_unpack(m, q, mask_bits, (hipStream_t)stream);
}

int cbk_gemv_batch(int n, const cbk_desc* descs, const void* const* xs, const int64_t* ldxs, int x_dtype, int M,
                   void* const* ys, const int64_t* ldys, int y_dtype, const void* const* biases,
                   void* workspace, size_t workspace_bytes, void* stream) {
  if (n < 1 || n > kMaxBatch) return CBK_ERR_SHAPE;
  if (!descs || !xs || !ldxs || !ys || !ldys) return CBK_ERR_NULL;
  if (M > 16) return CBK_ERR_SHAPE;
  const size_t ysz = y_dtype == CBK_F32 ? 4 : 2;
  GvCall calls[kMaxBatch];
  int nc = 0;
  bool fast = true;
  for (int i = 0; i < n; ++i) {
    GvCall c;
    int rc = to_dmat(descs + i, &c.m, true);
    if (rc) return rc;
    rc = check_io(xs[i], x_dtype, M, ldxs[i], ys[i], y_dtype, ldys[i], c.m.N, c.m.K);
    if (rc) return rc;
    c.x = xs[i]; c.ldx = ldxs[i]; c.y = ys[i]; c.ldy = ldys[i];
    c.bias = biases ? biases[i] : nullptr;
    c.par = 0;
    GvCall sub[3];
    const int k = fast ? expand_fused(c, ysz, sub) : 0;
    if (k == 0 || nc + k > kMaxBatch) { fast = false; continue; }
    for (int j = 0; j < k; ++j) calls[nc++] = sub[j];
  }
  // activation rows per pass: as many (8, 4, 2 or 1) as the kernel takes for every matrix and
  // their digits fit in LDS with; a gate/up matrix stages two scaled copies of every activation row
  const int vm = fast && calls[0].par ? 2 : 1;
  int mc = M * vm > 4 ? 8 / vm : (M * vm > 2 ? 4 / vm : (M * vm >= 2 ? 2 / vm : 1));   // (three rows: one pass of four)
  for (int i = 0; fast && i < nc; ++i) {
    while (mc > 1 && !gemv_fast_takes(calls[i].m, mc * vm) && gemv_fast_takes(calls[i].m, vm)) mc >>= 1;
    fast = gemv_fast_takes(calls[i].m, vm) && gemv_same_config(calls[0].m, calls[i].m) && calls[i].par == calls[0].par;
  }
  hipStream_t st = (hipStream_t)stream;
  if (fast) {
    for (int m0 = 0, mp; m0 < M; m0 += mp) {            // the weights are streamed once per pass
      mp = M - m0 < mc ? M - m0 : mc;
      GvCall part[kMaxBatch];
      for (int i = 0; i < nc; ++i) {
        part[i] = calls[i];
        part[i].x = (const uint8_t*)calls[i].x + (size_t)m0 * calls[i].ldx * 2;
        part[i].y = (uint8_t*)calls[i].y + (size_t)m0 * calls[i].ldy * ysz;
      }
      int rc = launch_gemv_fast_batch(nc, part, x_dtype, mp, y_dtype, workspace, workspace_bytes, st);
      if (rc) return rc;
    }
    return CBK_OK;
  }
  if (n == 1) {
    DMat m;
    to_dmat(descs, &m, true);
    return launch_gemv_generic(m, xs[0], x_dtype, M, ldxs[0], ys[0], y_dtype, ldys[0], biases ? biases[0] : nullptr,
                               workspace, workspace_bytes, st);
  }
  // mixed or unsupported configurations: one matrix at a time
  size_t off = 0;
  for (int i = 0; i < n; ++i) {
    // (cbk_gemv uses a workspace where it has one and computes the same bits without)
    const size_t need = cbk_workspace_bytes(descs + i, M);
    const bool room = need && workspace && off + need <= workspace_bytes;
    int rc = cbk_gemv(descs + i, xs[i], x_dtype, M, ldxs[i], ys[i], y_dtype, ldys[i], biases ? biases[i] : nullptr,
                      room ? (uint8_t*)workspace + off : nullptr, room ? need : 0, stream);
    if (rc) return rc;
    if (room) off += need;
  }
  return CBK_OK;
}

int cbk_gemv(const cbk_desc* in, const void* x, int x_dtype, int M, int64_t ldx, void* y, int y_dtype,
             int64_t ldy, const void* bias, void* workspace, size_t workspace_bytes, void* stream) {
  DMat m;
  int rc = to_dmat(in, &m, true);
  if (rc) return rc;
  rc = check_io(x, x_dtype, M, ldx, y, y_dtype, ldy, m.N, m.K);
  if (rc) return rc;
  if (M > 16) return CBK_ERR_SHAPE;
  return cbk_gemv_batch(1, in, &x, &ldx, x_dtype, M, &y, &ldy, y_dtype, &bias, workspace, workspace_bytes, stream);
}

int cbk_gemm(const cbk_desc* in, const void* x, int x_dtype, int M, int64_t ldx, void* y, int y_dtype,
             int64_t ldy, const void* bias, void* workspace, size_t workspace_bytes, void* stream) {
  DMat m;
  int rc = to_dmat(in, &m, true);
  if (rc) return rc;
  rc = check_io(x, x_dtype, M, ldx, y, y_dtype, ldy, m.N, m.K);
  if (rc) return rc;
  if (family_of(m.layout) == FAM_SPARSE) {
    if (M <= 16)                                                    // not worth re-packing: the row kernel
      return cbk_gemv(in, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, workspace, workspace_bytes, stream);
    const Transient t = transient_dense4(m);
    const bool room = workspace && !((uintptr_t)workspace & 255) &&
                      workspace_bytes >= t.end + gemm_big_workspace(dense4_view(m, nullptr, t), M);
    if (!sparse_repackable(m) || !room) {
      // zero points that are no 4-bit codes, row-fused column scales, or no room for the dense
      // image: the row kernel, sixteen activation rows per pass, without a workspace
      const size_t ysz = y_dtype == CBK_F32 ? 4 : 2;
      for (int m0 = 0; m0 < M; m0 += 16) {
        const int mc = M - m0 < 16 ? M - m0 : 16;
        rc = cbk_gemv(in, (const uint8_t*)x + (size_t)m0 * ldx * 2, x_dtype, mc, ldx,
                      (uint8_t*)y + (size_t)m0 * ldy * ysz, y_dtype, ldy, bias, nullptr, 0, stream);
        if (rc) return rc;
      }
      return CBK_OK;
    }
    uint8_t* ws = (uint8_t*)workspace;
    const DMat d = dense4_view(m, ws, t);
    rc = launch_unpack(m, ws + t.q, ws + t.mask, (hipStream_t)stream);
    if (rc) return rc;
    rc = launch_pack(d, ws + t.mask, ws + t.q, m.scale, m.zero, 0, 0, nullptr, (hipStream_t)stream);
    if (rc) return rc;
    return launch_gemm_big(d, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, ws + t.end, workspace_bytes - t.end,
                           (hipStream_t)stream);
  }
  if (gemm_big_takes(m, M))
    return launch_gemm_big(m, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, workspace, workspace_bytes,
                           (hipStream_t)stream);
  int lo[3], hi[3], row[3];
  const int nr = fused_ranges(m, lo, hi, row);
  if (nr) {
    // q|k|v: each range is a matrix with one col_scale vector; the launches share the
    // workspace (pre-scaled activations), which the stream order keeps apart
    const size_t ysz = y_dtype == CBK_F32 ? 4 : 2;
    for (int i = 0; i < nr; ++i) {
      const DMat s = row_range(m, lo[i], hi[i], row[i]);
      rc = launch_gemm_big(s, x, x_dtype, M, ldx, (uint8_t*)y + (size_t)lo[i] * ysz, y_dtype, ldy,
                           bias ? (const uint8_t*)bias + (size_t)lo[i] * ysz : nullptr, workspace, workspace_bytes,
                           (hipStream_t)stream);
      if (rc) return rc;
    }
    return CBK_OK;
  }
  return launch_gemm(m, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, (hipStream_t)stream);
}

}  // extern "C"

// ------------------------------------------------------------------ cbk_gemm without a workspace argument
// Scratch of cbk_gemm_static: the pre-scaled activations and the partial output tiles that
// cbk_gemm keeps in the caller's workspace.  One copy per GPU, at its own address on each; in
// host code the name of the array is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) unsigned char scratch[CBK_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mu;
void* scratch_ptr[kMaxDevices];          // device address of `scratch` on every GPU seen so far

// The address of this GPU's copy of the array (looked up once per device, with that device
// current: the caller's), or nullptr if the runtime refuses.
void* scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> g(scratch_mu);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    scratch_ptr[dev] = p;
  }
  return scratch_ptr[dev];
}
}  // namespace

extern "C" {

int cbk_gemm_static(const cbk_desc* in, const void* x, int x_dtype, int M, int64_t ldx, void* y, int y_dtype,
                    int64_t ldy, const void* bias, void* stream) {
  if (cbk_workspace_bytes(in, M) > (size_t)CBK_STATIC_SCRATCH_BYTES) {
    DMat m;
    const int rc = to_dmat(in, &m, true);
    return rc ? rc : CBK_ERR_WORKSPACE;                             // more scratch than the array holds
  }
  void* ws = scratch_of_current_device();
  if (!ws) return CBK_ERR_HIP;
  return cbk_gemm(in, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, ws, (size_t)CBK_STATIC_SCRATCH_BYTES, stream);
}

int cbk_linear(const cbk_desc* in, const void* x, int x_dtype, int M, int64_t ldx, void* y, int y_dtype,
               int64_t ldy, const void* bias, void* workspace, size_t workspace_bytes, void* stream) {
  // up to 8 rows (one or two passes of the decode kernel) the weights are streamed faster than the
  // prefill kernel's 64-token tile decodes them (14336 x 4096: 28 us against 31 us; 54 us at 16 rows)
  if (M <= 8) return cbk_gemv(in, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, workspace, workspace_bytes, stream);
  // (the variable-length layouts have no matrix-core path of their own: cbk_gemm sends them to the
  // row kernel or re-packs them for the call)
  return cbk_gemm(in, x, x_dtype, M, ldx, y, y_dtype, ldy, bias, workspace, workspace_bytes, stream);
}

// Where cbk_linear_act keeps t = x . W_hat^T: float32 up to 128 activation rows, else the output type.
static int act_mid_dtype(int M, int y_dtype) { return M <= 128 ? CBK_F32 : y_dtype; }
static size_t act_mid_bytes(int K, int M, int y_dtype) {
  const size_t b = (size_t)M * K * (act_mid_dtype(M, y_dtype) == CBK_F32 ? 4 : 2);
  return (b + 255) & ~(size_t)255;
}

size_t cbk_linear_act_workspace_bytes(const cbk_desc* in, int M, int y_dtype) {
  cbk_desc d;
  if (M < 1 || canon(in, &d)) return 0;
  return act_mid_bytes(d.K, M, y_dtype) + cbk_workspace_bytes(in, M);
}

int cbk_linear_act(const cbk_desc* in, const void* x, int x_dtype, int M, int64_t ldx, void* y, int y_dtype,
                   int64_t ldy, const void* bias, int act, void* workspace, size_t workspace_bytes, void* stream) {
  DMat m;
  int rc = to_dmat(in, &m, true);
  if (rc) return rc;
  if (m.K & 1) return CBK_ERR_SHAPE;
  if (act != CBK_ACT_GELU_TANH && act != CBK_ACT_SILU) return CBK_ERR_UNSUPPORTED;
  if (y_dtype != CBK_F32 && y_dtype != CBK_F16 && y_dtype != CBK_BF16T) return CBK_ERR_DTYPE;
  if (!y) return CBK_ERR_NULL;
  if (M < 1 || ldy < m.K / 2) return CBK_ERR_SHAPE;
  if ((uintptr_t)y & (y_dtype == CBK_F32 ? 3 : 1)) return CBK_ERR_ALIGN;
  const size_t mid = act_mid_bytes(m.K, M, y_dtype);
  if (!workspace || ((uintptr_t)workspace & 255) || workspace_bytes < mid + cbk_workspace_bytes(in, M))
    return CBK_ERR_WORKSPACE;
  const int tdt = act_mid_dtype(M, y_dtype);
  if (M > 8 && m.cs_rows == 2 && gemm_big_takes(m, M)) {
    // the tile kernel leaves t as two halves (gate outputs, then up outputs): a workgroup holds
    // one parity of the rows, and interleaved it could only store single elements
    rc = check_io(x, x_dtype, M, ldx, workspace, tdt, m.K, m.N, m.K);
    if (rc) return rc;
    rc = launch_gemm_big(m, x, x_dtype, M, ldx, workspace, tdt, m.K, nullptr, (uint8_t*)workspace + mid,
                         workspace_bytes - mid, (hipStream_t)stream, true);
    if (rc) return rc;
    return launch_act_mul(workspace, tdt, m.K, y, y_dtype, ldy, M, m.K / 2, act, bias, (hipStream_t)stream, true);
  }
  rc = cbk_linear(in, x, x_dtype, M, ldx, workspace, tdt, m.K, nullptr, (uint8_t*)workspace + mid,
                  workspace_bytes - mid, stream);                  // the activation kernel adds the bias
  if (rc) return rc;
  return launch_act_mul(workspace, tdt, m.K, y, y_dtype, ldy, M, m.K / 2, act, bias, (hipStream_t)stream);
}

}  // extern "C"
