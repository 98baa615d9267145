// Prefill GEMM: activation pre-scaling kernel, the generic-reader instantiation
// and the dispatch over the per-code-width instantiations (cbk_gemm_big_b2/3/4.hip).  The
// kernel itself is in cbk_gemm_big.h.
#include "cbk_gemm_big.h"

namespace cbk {

int launch_gemm_big_b2(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b3(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b4(const GbArgs&, int keep, int group, int blocks, hipStream_t);
int launch_gemm_big_b6(const GbArgs&, int blocks, hipStream_t);

// ---- X' = fp16(x * col_scale / s_row), [Mpad, Npad] row-major, and s_row, one workgroup per row.
// s_row is the power of two that brings the row's largest |x * col_scale| below 2^15 (1 for
// nearly every row: only magnitudes beyond fp16's range need it); the GEMM kernel multiplies the
// row's outputs by it.  Rows M..Mpad-1 and columns N..Npad-1 are zero.
__device__ inline void prep8(const uint4 v, const uint4 c, int xdt, float (&a)[8]) {
  const uint32_t xw[4] = {v.x, v.y, v.z, v.w}, cw[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (xdt == CBK_F16) { a[2 * e] = h2f((uint16_t)(xw[e] & 0xffffu)); a[2 * e + 1] = h2f((uint16_t)(xw[e] >> 16)); }
    else { a[2 * e] = bf2f((uint16_t)(xw[e] & 0xffffu)); a[2 * e + 1] = bf2f((uint16_t)(xw[e] >> 16)); }
    a[2 * e] *= h2f((uint16_t)(cw[e] & 0xffffu)); a[2 * e + 1] *= h2f((uint16_t)(cw[e] >> 16));
  }
}

// One workgroup of 1024 threads per row.  CH: 16-byte pieces of the row a thread keeps in
// registers between the two passes (the row is read from memory once); 0 = any row length, the
// second pass reads the row again.
template <int CH>
__global__ __launch_bounds__(1024) void gemm_prep_kernel(const uint16_t* x, int64_t ldx, const uint16_t* cs, int xdt,
                                                         int M, int N, int Npad, uint16_t* out, float* row_scale) {
  constexpr int T = 1024;
  __shared__ float red[T / 64];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int n8 = Npad >> 3, nv = N >> 3;                           // N is a multiple of 128
  uint16_t* orow = out + (size_t)row * Npad;
  if (row >= M) {
    for (int c8 = tid; c8 < n8; c8 += T) *(uint4*)(orow + c8 * 8) = make_uint4(0, 0, 0, 0);
    if (tid == 0) row_scale[row] = 1.f;
    return;
  }
  const uint16_t* xr = x + (size_t)row * ldx;
  const uint4 one = make_uint4(0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u);
  uint4 xv[CH ? CH : 1], cv[CH ? CH : 1];
  float mx = 0.f;
  if (CH) {
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int c8 = tid + T * i;
      xv[i] = make_uint4(0, 0, 0, 0); cv[i] = one;
      if (c8 < nv) { xv[i] = *(const uint4*)(xr + c8 * 8); if (cs) cv[i] = *(const uint4*)(cs + c8 * 8); }
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      float a[8];
      prep8(xv[i], cv[i], xdt, a);
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(a[e]));
    }
  } else {
    for (int c8 = tid; c8 < nv; c8 += T) {
      float a[8];
      prep8(*(const uint4*)(xr + c8 * 8), cs ? *(const uint4*)(cs + c8 * 8) : one, xdt, a);
#pragma unroll
      for (int e = 0; e < 8; ++e) mx = fmaxf(mx, fabsf(a[e]));
    }
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  if ((tid & 63) == 0) red[tid >> 6] = mx;
  __syncthreads();
  float all = red[0];
#pragma unroll
  for (int w = 1; w < T / 64; ++w) all = fmaxf(all, red[w]);
  const float s = token_scale(all);
  const float inv = 1.f / s;                                       // a power of two: exact
  if (tid == 0) row_scale[row] = s;
  auto emit = [&](int c8, const uint4 xq, const uint4 cq) {
    uint4 o4 = make_uint4(0, 0, 0, 0);
    if (c8 < nv) {
      float a[8];
      prep8(xq, cq, xdt, a);
      uint32_t o[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (uint32_t)f2h(a[2 * e] * inv) | ((uint32_t)f2h(a[2 * e + 1] * inv) << 16);
      o4 = make_uint4(o[0], o[1], o[2], o[3]);
    }
    *(uint4*)(orow + c8 * 8) = o4;
  };
  if (CH) {
#pragma unroll
    for (int i = 0; i < CH; ++i)
      if (tid + T * i < n8) emit(tid + T * i, xv[i], cv[i]);
  } else {
    for (int c8 = tid; c8 < n8; c8 += T)
      emit(c8, c8 < nv ? *(const uint4*)(xr + c8 * 8) : one, (cs && c8 < nv) ? *(const uint4*)(cs + c8 * 8) : one);
  }
}

static inline int gb_npad(int N) { return (N + 255) / 256 * 256; }

// ---- y = sum of the float32 partial tiles (+ bias), eight outputs per thread
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(const float* part, size_t part_stride, int64_t part_ld,
                                                               int nsplit, int M, int K, const void* bias, void* y,
                                                               int ydt, int64_t ldy) {
  const int k8 = (K + 7) >> 3;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)M * k8) return;
  const int tok = (int)(id / k8), k0 = (int)(id % k8) * 8;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = 0.f;
  for (int p = 0; p < nsplit; ++p) {                                // fixed order: run-to-run identical
    const float* src = part + (size_t)p * part_stride + (size_t)tok * part_ld + k0;
    const float4 a = ((const float4*)src)[0], b = ((const float4*)src)[1];
    v[0] += a.x; v[1] += a.y; v[2] += a.z; v[3] += a.w; v[4] += b.x; v[5] += b.y; v[6] += b.z; v[7] += b.w;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int k = k0 + e;
    if (k >= K) break;
    float o = v[e];
    if (bias) o += ydt == CBK_F32 ? ((const float*)bias)[k] : ydt == CBK_F16 ? h2f(((const uint16_t*)bias)[k]) : bf2f(((const uint16_t*)bias)[k]);
    const size_t at = (size_t)tok * ldy + k;
    if (ydt == CBK_F32) ((float*)y)[at] = o;
    else if (ydt == CBK_F16) ((uint16_t*)y)[at] = f2h(o);
    else ((uint16_t*)y)[at] = f2bf(o);
  }
}

// the matrices the byte-permute instantiations take (the others go through the generic reader,
// whose launches are never split)
static bool gb_fast(const DMat& m) {
  const int fam = family_of(m.layout);
  if (!(m.flags & CBK_FLAG_ZERO_LE_128) || (m.group != 64 && m.group != 128)) return false;
  if (fam == FAM_BLK6) return m.bits == 6 && m.keep == 16 && m.group == 128;
  if (m.bits < 2 || m.bits > 4) return false;
  if (fam == FAM_BLK) return m.keep == 10 || m.keep == 16 || m.keep == 23;
  return fam == FAM_DENSE;
}

// Token tile and split of the column range of a call.
//  * A launch of fewer tiles than a multiple of the 256 CUs leaves CUs idle for a whole tile
//    time; cutting the column range over several workgroups per output tile gives them work at
//    the price of the float32 partial tiles (written and read once).
//  * Calls of at most 64 / 128 activation rows take the 64- / 128-token tile.  Larger calls
//    take the 256-token tile unless the model below gives the 128-token tile the shorter time,
//    which it does for small matrices (4096 x 4096 at 256 to 2048 rows: 16 to 128 tiles of 256
//    tokens): twice the tiles, each 0.8 of the time.
// Times in microseconds from measurements of this kernel: per 64-column stage 1.1 / 1.35 / 1.7
// for the three tiles (the 64-token stage is bound by the weight loads' latency), 8 - 10 per
// workgroup outside the stage loop, 4 TB/s for the partial tiles.  Over 24 measured calls
// (eight shapes, 256 / 512 / 2048 rows) the choice is within 2 % of the faster tile; always
// taking the 256-token tile loses 6 % on average and up to 34 %.
struct GbPlan { int ti, nsplit; double t; };
static GbPlan gb_plan_ti(const DMat& m, int M, int ti) {
  const int T = 64 * ti;
  const int tiles = ((M + T - 1) / T) * ((m.K + GB_R - 1) / GB_R);
  const int nst = gb_npad(m.N) / GB_K;
  const double t_stage = ti == 1 ? 1.1 : ti == 2 ? 1.35 : 1.7, t_wg = ti == 1 ? 8.0 : 10.0;
  GbPlan best{ti, 1, 0.0};
  double t1 = 0;
  const bool may_split = m.cs_rows <= 1 && gb_fast(m);
  for (int s = 1; s <= (may_split ? 16 : 1); ++s) {
    const int per = ((nst + s - 1) / s + 3) / 4 * 4;                // stages per part, a multiple of 4
    if (s > 1 && (s - 1) * per >= nst) continue;                    // a part would be empty
    const double rounds = (double)((tiles * s + 255) / 256);
    double t = rounds * (per * t_stage + t_wg);
    if (s > 1) t += 2.0 * s * (double)M * m.K * 4 / 4.0e6 + 5.0;
    if (s == 1) { t1 = t; best.t = t; }
    else if (t < best.t) { best.nsplit = s; best.t = t; }
  }
  if (best.t > 0.93 * t1) { best.nsplit = 1; best.t = t1; }         // not worth a second kernel
  return best;
}
static GbPlan gb_plan(const DMat& m, int M) {
  if (M <= 64) return gb_plan_ti(m, M, 1);
  if (M <= 128) return gb_plan_ti(m, M, 2);
  const GbPlan p4 = gb_plan_ti(m, M, 4), p2 = gb_plan_ti(m, M, 2);
  return p2.t < p4.t ? p2 : p4;
}

static inline size_t gb_kpad(int K) { return (size_t)(K + 7) / 8 * 8; }

size_t gemm_big_workspace(const DMat& m, int M) {
  const GbPlan plan = gb_plan(m, M);
  const size_t T = 64 * plan.ti, mpad = (size_t)(M + T - 1) / T * T;
  const size_t nv = m.cs_rows > 1 ? m.cs_rows : 1;
  size_t b = (nv * mpad * gb_npad(m.N) * 2 + 255) & ~(size_t)255;     // X', one per col_scale vector
  b += (nv * mpad * 4 + 255) & ~(size_t)255;                          // and its row scales
  const int ns = plan.nsplit;
  if (ns > 1) b += ((size_t)ns * M * gb_kpad(m.K) * 4 + 255) & ~(size_t)255;
  return b;
}

// halves: a gate/up matrix's outputs as two halves of y (GbArgs::halves) instead of interleaved
int launch_gemm_big(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                    const void* bias, void* ws, size_t ws_bytes, hipStream_t st, bool halves) {
  if (halves && (m.cs_rows != 2 || (m.K & 1) || bias)) return CBK_ERR_UNSUPPORTED;
  if (family_of(m.layout) == FAM_SPARSE) return CBK_ERR_UNSUPPORTED;
  // q|k|v ranges off the row-tile grid: the caller passes them one by one
  if (m.cs_rows == 3 && (m.cs_split0 % GB_R || (m.cs_split0 + m.cs_split1) % GB_R)) return CBK_ERR_UNSUPPORTED;
  if (ydt != CBK_F32 && ydt != CBK_F16 && ydt != CBK_BF16T) return CBK_ERR_DTYPE;
  if (!ws || ws_bytes < gemm_big_workspace(m, M)) return CBK_ERR_WORKSPACE;
  if ((uintptr_t)ws & 255) return CBK_ERR_ALIGN;
  const GbPlan plan = gb_plan(m, M);
  const int T = 64 * plan.ti;
  const int Mpad = (M + T - 1) / T * T;
  const int Npad = gb_npad(m.N);
  const int par = m.cs_rows == 2 ? 1 : 0;
  const int nv = m.cs_rows > 1 ? m.cs_rows : 1;
  const size_t xbytes = ((size_t)nv * Mpad * Npad * 2 + 255) & ~(size_t)255;
  const size_t sbytes = ((size_t)nv * Mpad * 4 + 255) & ~(size_t)255;
  float* row_scale = (float*)((uint8_t*)ws + xbytes);
  const int ch = (Npad / 8 + 1023) / 1024;                         // 16-byte pieces per thread of the row kernel
  auto prep = ch <= 1 ? gemm_prep_kernel<1> : ch <= 3 ? gemm_prep_kernel<3> : gemm_prep_kernel<0>;
  for (int v = 0; v < nv; ++v)                                     // one X' per col_scale vector
    hipLaunchKernelGGL(prep, dim3((unsigned)Mpad), dim3(1024), 0, st,
                       (const uint16_t*)x, ldx, m.cs ? m.cs + (size_t)v * m.N : nullptr, xdt, M, m.N, Npad,
                       (uint16_t*)ws + (size_t)v * Mpad * Npad, row_scale + (size_t)v * Mpad);
  GbArgs a;
  a.m = m; a.xp = (const uint16_t*)ws; a.M = M; a.Npad = Npad; a.y = y; a.ydt = ydt; a.ldy = ldy; a.bias = bias;
  a.par = par; a.xps = (size_t)Mpad * Npad;
  a.halves = halves ? 1 : 0;
  a.row_scale = row_scale; a.rss = Mpad;
  a.vs0 = m.cs_rows == 3 ? m.cs_split0 : 0x7fffffff;
  a.vs1 = m.cs_rows == 3 ? m.cs_split0 + m.cs_split1 : 0x7fffffff;
  const int nst_all = Npad / GB_K;
  a.nsplit = plan.nsplit;
  a.nst_part = ((nst_all + a.nsplit - 1) / a.nsplit + 3) / 4 * 4;
  a.part_ld = (int64_t)gb_kpad(m.K);
  a.part_stride = (size_t)M * gb_kpad(m.K);
  a.part = (float*)((uint8_t*)ws + xbytes + sbytes);
  a.ti = plan.ti;
  a.tiles_t = (M + T - 1) / T;
  a.tiles_r = par ? 2 * ((m.K + 2 * GB_R - 1) / (2 * GB_R)) : (m.K + GB_R - 1) / GB_R;
  const int nb = a.tiles_t * a.tiles_r * a.nsplit;
  const int blocks = ((nb + 7) / 8) * 8;
  const bool le128 = (m.flags & CBK_FLAG_ZERO_LE_128) != 0;
  const int fam = family_of(m.layout);
  int rc = CBK_ERR_UNSUPPORTED;
  if (le128 && (fam == FAM_BLK || fam == FAM_DENSE)) {
    const int keep = fam == FAM_DENSE ? 0 : m.keep;
    if (m.bits == 2) rc = launch_gemm_big_b2(a, keep, m.group, blocks, st);
    else if (m.bits == 3) rc = launch_gemm_big_b3(a, keep, m.group, blocks, st);
    else if (m.bits == 4) rc = launch_gemm_big_b4(a, keep, m.group, blocks, st);
  } else if (le128 && fam == FAM_BLK6 && m.bits == 6 && m.keep == 16 && m.group == 128) {
    rc = launch_gemm_big_b6(a, blocks, st);
  }
  if (rc == CBK_ERR_UNSUPPORTED) {
    if (a.nsplit > 1) return CBK_ERR_UNSUPPORTED;                   // (only what the cases above take is ever split)
    rc = launch_big_cfg<0, 0, 128>(a, blocks, st);                  // generic reader
  }
  if (rc == CBK_OK && a.nsplit > 1) {
    const int64_t items = (int64_t)M * ((m.K + 7) / 8);
    hipLaunchKernelGGL(gemm_split_reduce_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st,
                       (const float*)a.part, a.part_stride, a.part_ld, a.nsplit, M, m.K, bias, y, ydt, ldy);
    if (hipGetLastError() != hipSuccess) rc = CBK_ERR_HIP;
  }
  return rc;
}

}  // namespace cbk
