/* CPU oracle for the CBK1 sparse low-bit linear layer, in C.  TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's dequantiser and of its dequantise-then-matmul
 * forward, written from the format text and independent of the numpy oracle next to it.  It
 * is loaded only by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
 * bench.py (where it is the thing timed on the host cores); the product library never links
 * or calls it.
 *
 * Reference files each function follows (paths relative to the reference checkout):
 *   keep bit, code planes     docs/FORMAT.md:83-122, src/cobaltkernel/dequant_ref.py:43-68,
 *                             src/cobaltkernel/pack_cobalt.py:155-250
 *   variable-length rows      src/cobaltkernel/pack_cobalt.py:201-250,
 *                             src/cobaltkernel/csrc/cobalt_format.h:70-75
 *   dequant formula           src/cobaltkernel/dequant_ref.py:69-103 (fp32, ((q-z)*s)*keep*cs)
 *   col_scale row choice      src/cobaltkernel/csrc/cobalt_format.h:77-99, dequant_ref.py:73-82
 *   forward                   benchmarks/benchmark_suite.py:1200-1217 (y = x @ W_hat.T + bias)
 *
 * Layout ids: 0 SPARSE4, 1 DENSE4, 2 DENSE8, 3 SPARSE4X, 5 SPARSE4E, 6 BLK1632_4,
 * 7 BLK1632_6 are the reference's; 8 BLKC (mask plane + LSB-first survivor bit stream,
 * `keep` survivors per 32 columns) and 9 DENSEB (LSB-first bit stream of every column) are
 * this build's extension for 2/3-bit codes and group 64.
 *
 * Parity status: pinned by tests/test_oracle_c.py, which checks it bit for bit against the
 * numpy oracle (itself pinned by hand-computed byte vectors and known answers) on every
 * layout, and against a float64 evaluation of the formula rounded once.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { SPARSE4 = 0, DENSE4 = 1, DENSE8 = 2, SPARSE4X = 3, SPARSE4E = 5, BLK1632_4 = 6, BLK1632_6 = 7,
       BLKC = 8, DENSEB = 9 };

static size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

/* IEEE binary16 bits -> float, exact (subnormals, infinities and NaN included) */
static float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
  uint32_t u;
  if (e == 0) {
    if (m == 0) u = sign;
    else {                                    /* subnormal: m * 2^-24 */
      float f = (float)m * 5.9604644775390625e-08f;
      memcpy(&u, &f, 4);
      u |= sign;
    }
  } else if (e == 31) u = sign | 0x7F800000u | (m << 13);
  else u = sign | ((e + 112u) << 23) | (m << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static int is_sparse(int layout) { return layout == SPARSE4 || layout == SPARSE4X || layout == SPARSE4E; }
static int is_dense(int layout) { return layout == DENSE4 || layout == DENSE8 || layout == DENSEB; }

/* canonical (bits, group, keep) of a layout; returns 0 if the combination is invalid */
static int canon(int layout, int* bits, int* group, int* keep) {
  switch (layout) {
    case DENSE4: *bits = 4; *group = 128; *keep = 0; return 1;
    case DENSE8: *bits = 8; *group = 128; *keep = 0; return 1;
    case SPARSE4: case SPARSE4X: case SPARSE4E: *bits = 4; *group = 128; *keep = 0; return 1;
    case BLK1632_4: *bits = 4; *group = 128; *keep = 16; return 1;
    case BLK1632_6: *bits = 6; *group = 128; *keep = 16; return 1;
    case BLKC:
      return (*bits == 2 || *bits == 3 || *bits == 4) && *keep >= 1 && *keep <= 32 && (*group == 64 || *group == 128);
    case DENSEB:
      *keep = 0;
      return (*bits == 2 || *bits == 3 || *bits == 4 || *bits == 8) && (*group == 64 || *group == 128);
    default: return 0;
  }
}

/* bytes per row of a fixed-stride layout (0 for the variable-length family) */
size_t cbk_ref_row_stride(int layout, int N, int bits, int group, int keep) {
  if (!canon(layout, &bits, &group, &keep)) return 0;
  if (is_sparse(layout)) return 0;
  if (is_dense(layout)) return align_up(((size_t)N * bits + 7) / 8, 16);
  if (layout == BLK1632_6) return (size_t)N / 2;
  return (size_t)N / 8 + align_up(((size_t)(N / 32) * keep * bits + 7) / 8, 16);
}

static uint32_t get_bits(const uint8_t* base, size_t bitpos, int nb) {
  uint32_t v = 0;
  for (int i = 0; i < nb; ++i) {
    const size_t p = bitpos + (size_t)i;
    v |= (uint32_t)((base[p >> 3] >> (p & 7)) & 1u) << i;
  }
  return v;
}

/* stored codes and keep flags of one row: q[j] (0 for a pruned column), kp[j] in {0,1} */
static void decode_row(const uint8_t* data, const uint32_t* row_off, int k, int N, int layout, int bits, int group,
                       int keep, int* q, uint8_t* kp) {
  const int G = N / group;
  if (is_dense(layout)) {
    const uint8_t* row = data + (size_t)k * cbk_ref_row_stride(layout, N, bits, group, keep);
    for (int j = 0; j < N; ++j) { q[j] = (int)get_bits(row, (size_t)j * bits, bits); kp[j] = 1; }
    return;
  }
  if (is_sparse(layout)) {
    const uint8_t* row = data + row_off[k];
    const int has_goff = layout != SPARSE4;
    const size_t hdr = align_up((size_t)N / 8 + (has_goff ? align_up((size_t)G * 2, 16) : 0), 16);
    size_t nib = 0;
    for (int j = 0; j < N; ++j) {
      if (j % group == 0 && (nib & 1)) ++nib;            /* every group starts on a byte boundary */
      kp[j] = (row[j >> 3] >> (j & 7)) & 1u;
      q[j] = 0;
      if (kp[j]) {
        const uint8_t b = row[hdr + (nib >> 1)];
        q[j] = (nib & 1) ? (b >> 4) : (b & 0xF);
        ++nib;
      }
    }
    return;
  }
  const uint8_t* row = data + (size_t)k * cbk_ref_row_stride(layout, N, bits, group, keep);
  size_t rank = 0;
  for (int j = 0; j < N; ++j) {
    kp[j] = (row[j >> 3] >> (j & 7)) & 1u;
    q[j] = 0;
    if (!kp[j]) continue;
    if (layout == BLK1632_6) {
      const size_t t = rank / 16, i = rank % 16;
      const uint8_t b = row[(size_t)N / 8 + 8 * t + (i >> 1)];
      const uint32_t lo = (i & 1) ? (b >> 4) : (b & 0xF);
      uint32_t hw;
      memcpy(&hw, row + 3 * (size_t)N / 8 + 4 * t, 4);   /* little-endian host */
      const uint32_t hi = (hw >> (2 * (i >> 1) + ((i & 1) ? 16 : 0))) & 3u;
      q[j] = (int)(lo | (hi << 4));
    } else {
      q[j] = (int)get_bits(row + (size_t)N / 8, rank * (size_t)bits, bits);
    }
    ++rank;
  }
}

static int cs_row_of(int k, int cs_rows, int split0, int split1) {
  if (cs_rows <= 1) return 0;
  if (cs_rows == 2) return k & 1;
  return k < split0 ? 0 : (k < split0 + split1 ? 1 : 2);
}

/* one row of W_hat: ((q - zero) * scale) * keep * col_scale, every step rounded to float32 */
static void dequant_one_row(const uint8_t* data, const uint32_t* row_off, const uint16_t* scale, const uint8_t* zero,
                            const uint16_t* col_scale, int k, int N, int layout, int bits, int group, int keep,
                            int cs_rows, int split0, int split1, int* q, uint8_t* kp, float* out) {
  const int G = N / group;
  decode_row(data, row_off, k, N, layout, bits, group, keep, q, kp);
  const uint16_t* cs = (col_scale && cs_rows > 0) ? col_scale + (size_t)cs_row_of(k, cs_rows, split0, split1) * N : 0;
  for (int j = 0; j < N; ++j) {
    const int g = j / group;
    const float s = half_bits_to_float(scale[(size_t)k * G + g]);
    const float z = (float)zero[(size_t)k * G + g];
    volatile float w = ((float)q[j] - z) * s;              /* volatile: one float32 rounding per step */
    if (!is_dense(layout)) w = w * (float)kp[j];
    if (cs) w = w * half_bits_to_float(cs[j]);
    out[j] = w;
  }
}

/* W_hat rows [row0, row0+nrows) as float32 [nrows, N].  scale / col_scale are binary16 bit
 * patterns.  Returns 0 on success. */
int cbk_ref_dequant(const uint8_t* data, const uint32_t* row_off, const uint16_t* scale, const uint8_t* zero,
                    const uint16_t* col_scale, int K, int N, int layout, int bits, int group, int keep,
                    int cs_rows, int split0, int split1, int row0, int nrows, float* out) {
  if (!canon(layout, &bits, &group, &keep) || N % 128 || row0 < 0 || row0 + nrows > K) return -1;
  int rc = 0;
#pragma omp parallel
  {
    int* q = (int*)__builtin_malloc((size_t)N * sizeof(int));
    uint8_t* kp = (uint8_t*)__builtin_malloc((size_t)N);
    if (!q || !kp) {
#pragma omp atomic write
      rc = -2;
    } else {
#pragma omp for schedule(static)
      for (int r = 0; r < nrows; ++r)
        dequant_one_row(data, row_off, scale, zero, col_scale, row0 + r, N, layout, bits, group, keep, cs_rows,
                        split0, split1, q, kp, out + (size_t)r * N);
    }
    __builtin_free(q);
    __builtin_free(kp);
  }
  return rc;
}

/* y[m, k] = sum_j x[m, j] * W_hat[k, j] (+ bias[k]), W_hat float32 as above, double accumulate.
 * x is [M, N] float32 (the caller widens fp16/bf16 exactly), y is [M, K] double. */
int cbk_ref_forward(const uint8_t* data, const uint32_t* row_off, const uint16_t* scale, const uint8_t* zero,
                    const uint16_t* col_scale, int K, int N, int layout, int bits, int group, int keep,
                    int cs_rows, int split0, int split1, const float* x, int M, const double* bias, double* y) {
  if (!canon(layout, &bits, &group, &keep) || N % 128) return -1;
  int rc = 0;
#pragma omp parallel
  {
    float* w = (float*)__builtin_malloc((size_t)N * sizeof(float));
    int* q = (int*)__builtin_malloc((size_t)N * sizeof(int));
    uint8_t* kp = (uint8_t*)__builtin_malloc((size_t)N);
    if (!w || !q || !kp) {
#pragma omp atomic write
      rc = -2;
    } else {
#pragma omp for schedule(static)
      for (int k = 0; k < K; ++k) {
        dequant_one_row(data, row_off, scale, zero, col_scale, k, N, layout, bits, group, keep, cs_rows, split0,
                        split1, q, kp, w);
        for (int m = 0; m < M; ++m) {
          double acc = 0.0;
          const float* xm = x + (size_t)m * N;
          for (int j = 0; j < N; ++j) acc += (double)xm[j] * (double)w[j];
          y[(size_t)m * K + k] = acc + (bias ? bias[k] : 0.0);
        }
      }
    }
    __builtin_free(w);
    __builtin_free(q);
    __builtin_free(kp);
  }
  return rc;
}

int cbk_ref_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void cbk_ref_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
