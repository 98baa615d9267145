// Reference-shaped decode GEMV for EVERY layout: one wavefront per weight row, lanes stride
// over 32-column blocks (fixed-stride layouts through the generic reader; the survivor streams
// with vector loads and a register nibble stream), float32 FMA, butterfly reduction.  It is the path for layouts and
// parameter combinations the MFMA decode kernel does not take (variable-length SPARSE4*,
// DENSE8, zero points above 127) and the yardstick the fast kernel is checked
// against.  Computes, per row k and activation row m,
//     y[m,k] = sum_g scale[k,g] * sum_{j in g, kept} (q[k,j] - zero[k,g]) * (x[m,j]*cs[j])
// which is the accumulation order of cbk::gemv_rows in the reference
// (src/cobaltkernel/csrc/cobalt_gemv.cuh:295,537,586) with the zero point applied per
// kept column, so a pruned column contributes exactly 0 whatever `zero` holds.
#include "cbk_device.h"

namespace cbk {

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

constexpr int SP4_MAX_G = 512;     // groups per row whose offsets the SPARSE4 path keeps in LDS (N <= 65536)

// PATH picks the reader at compile time (one kernel per reader keeps each one's register count,
// and with it the number of resident wavefronts, its own): 0 DENSE8, 1 the other fixed-stride
// layouts, 2 survivor streams with group offsets at hand, 3 SPARSE4 rows with more groups than
// the offset table holds.
template <int XDT, int M, int PATH>
__global__ __launch_bounds__(256) void gemv_generic_kernel(DMat m, const void* x, int64_t ldx, void* y,
                                                           int ydt, int64_t ldy, const void* bias) {
  __shared__ uint32_t sp4_goff[PATH == 2 ? 4 * SP4_MAX_G : 4];
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int nwaves = (gridDim.x * blockDim.x) >> 6;
  for (int k = wave; k < m.K; k += nwaves) {
    float acc[M];
#pragma unroll
    for (int i = 0; i < M; ++i) acc[i] = 0.f;
    const uint16_t* cs = m.cs ? m.cs + (size_t)cs_row_of(m, k) * m.N : nullptr;
    if constexpr (PATH == 0) {
      // one byte per column: a lane takes a 32-column block as two 16-byte units of codes and
      // whole vectors of activations and column scales
      const RowView row = row_view(m, k);
      for (int t = lane; t < m.N / BLOCK; t += 64) {
        const uint4 c0 = *(const uint4*)row.unit(2 * t), c1 = *(const uint4*)row.unit(2 * t + 1);
        const uint32_t cw[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const int g = (t * BLOCK) / m.group;
        const float s = h2f(m.scale[meta_index(m, k, g)]);
        const float z = (float)m.zero[meta_index(m, k, g)];
        float part[M];
#pragma unroll
        for (int i = 0; i < M; ++i) part[i] = 0.f;
#pragma unroll
        for (int o = 0; o < 4; ++o) {                               // eight columns at a time
          const int col = t * BLOCK + 8 * o;
          float wv[8];
#pragma unroll
          for (int p = 0; p < 8; ++p) wv[p] = (float)((cw[2 * o + (p >> 2)] >> (8 * (p & 3))) & 0xFFu) - z;
          if (cs) {
            const uint4 cv = *(const uint4*)(cs + col);
            const uint32_t sw[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
            for (int p = 0; p < 8; ++p) wv[p] *= h2f((uint16_t)(sw[p >> 1] >> (16 * (p & 1))));
          }
#pragma unroll
          for (int i = 0; i < M; ++i) {
            const uint4 xv = *(const uint4*)((const uint16_t*)x + (size_t)i * ldx + col);
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int p = 0; p < 8; ++p) {
              const uint16_t hb = (uint16_t)(xw[p >> 1] >> (16 * (p & 1)));
              part[i] = fmaf(wv[p], XDT == CBK_F16 ? h2f(hb) : bf2f(hb), part[i]);
            }
          }
        }
#pragma unroll
        for (int i = 0; i < M; ++i) acc[i] = fmaf(s, part[i], acc[i]);
      }
    } else if constexpr (PATH == 1) {
      const RowView row = row_view(m, k);
      for (int t = lane; t < m.N / BLOCK; t += 64) {
        int q[32];
        const uint32_t keep = decode_block32(m, row, t, q);
        const int g = (t * BLOCK) / m.group;
        const float s = h2f(m.scale[meta_index(m, k, g)]);
        const int z = m.zero[meta_index(m, k, g)];
        float part[M];
#pragma unroll
        for (int i = 0; i < M; ++i) part[i] = 0.f;
#pragma unroll
        for (int p = 0; p < 32; ++p) {
          const int col = t * BLOCK + p;
          const float w = ((keep >> p) & 1u) ? (float)(q[p] - z) : 0.f;
          const float c = cs ? h2f(cs[col]) : 1.f;
#pragma unroll
          for (int i = 0; i < M; ++i)
            part[i] = fmaf(w, load_act<XDT>(x, (size_t)i * ldx + col) * c, part[i]);
        }
#pragma unroll
        for (int i = 0; i < M; ++i) acc[i] = fmaf(s, part[i], acc[i]);
      }
    } else if constexpr (PATH == 2) {
      // The byte offset of every group's codes is in the row's header (SPARSE4X / SPARSE4E) or
      // is summed up here from the bitmap (SPARSE4: a prefix sum of the groups' byte counts over
      // the wavefront, kept in LDS), so a lane can take one 32-column block: its survivors'
      // nibbles start popc(earlier blocks of the group) nibbles into the group.  Activations, column scales and the (at most 17) code
      // bytes are fetched up front as whole vectors; the nibbles are then shifted out of a
      // register stream under the mask bits, one mask byte at a time.
      const uint8_t* row = m.data + m.row_off[k];
      const uint32_t* bm = (const uint32_t*)row;
      const bool has_goff = m.layout != CBK_SPARSE4;
      const int hdr = ((m.N >> 3) + (has_goff ? ((m.G * 2 + 15) & ~15) : 0) + 15) & ~15;
      const uint16_t* goff = (const uint16_t*)(row + (m.N >> 3));
      uint32_t* lgoff = sp4_goff + (threadIdx.x >> 6) * SP4_MAX_G;
      if (!has_goff) {
        uint32_t carry = 0;
        for (int g0 = 0; g0 < m.G; g0 += 64) {
          const int g = g0 + lane;
          uint32_t nb = 0;                                          // bytes of group g: an even number of nibbles
          if (g < m.G) nb = (uint32_t)(__popc(bm[4 * g]) + __popc(bm[4 * g + 1]) + __popc(bm[4 * g + 2]) + __popc(bm[4 * g + 3]) + 1) >> 1;
          uint32_t incl = nb;
#pragma unroll
          for (int o = 1; o < 64; o <<= 1) {
            const uint32_t v = (uint32_t)__shfl_up((int)incl, o, 64);
            incl += lane >= o ? v : 0u;
          }
          if (g < m.G) lgoff[g] = carry + incl - nb;
          carry += (uint32_t)__shfl((int)incl, 63, 64);
        }
        __builtin_amdgcn_wave_barrier();
      }
      for (int t = lane; t < m.N / BLOCK; t += 64) {
        const int g = t >> 2, j = t & 3;
        const uint32_t mw = bm[t];
        uint32_t pre = 0;                                           // nibbles of the group before this block
        if (j > 0) pre += __popc(bm[4 * g]);
        if (j > 1) pre += __popc(bm[4 * g + 1]);
        if (j > 2) pre += __popc(bm[4 * g + 2]);
        const uint8_t* cp = row + hdr + (has_goff ? (uint32_t)goff[g] : lgoff[g]) + (pre >> 1);
        const uintptr_t ca = (uintptr_t)cp & ~(uintptr_t)3;
        const uint32_t sh = (uint32_t)(((uintptr_t)cp & 3) * 8 + (pre & 1) * 4);   // < 32
        uint32_t e[6];
#pragma unroll
        for (int i = 0; i < 6; ++i) e[i] = ((const uint32_t*)ca)[i];               // 17 bytes + skew; rows end in a readable tail
        uint32_t w[5];
#pragma unroll
        for (int i = 0; i < 5; ++i) w[i] = __builtin_amdgcn_alignbit(e[i + 1], e[i], sh);
        const float s = h2f(m.scale[(size_t)k * m.G + g]);
        const float z = (float)m.zero[(size_t)k * m.G + g];
        float part[M];
#pragma unroll
        for (int i = 0; i < M; ++i) part[i] = 0.f;
#pragma unroll
        for (int jb = 0; jb < 4; ++jb) {
          const uint32_t mb = (mw >> (8 * jb)) & 0xFFu;
          const uint32_t r = jb == 0 ? 0u : (uint32_t)__popc(mw & ((1u << (8 * jb)) - 1u));     // survivors before this byte
          // 32 bits of the stream from nibble r on: dword r / 8 and the next one, picked by selects
          const uint32_t idx = r >> 3, bs = (r & 7u) * 4u;
          uint32_t lo = w[0], hi = w[1];
#pragma unroll
          for (int i = 1; i < 4; ++i) { lo = idx == (uint32_t)i ? w[i] : lo; hi = idx == (uint32_t)i ? w[i + 1] : hi; }
          lo = idx >= 4u ? w[4] : lo; hi = idx >= 4u ? 0u : hi;
          uint32_t win = __builtin_amdgcn_alignbit(hi, lo, bs);
          const int c0 = t * BLOCK + 8 * jb;
          float cf[8];
          if (cs) {
            const uint4 cv = *(const uint4*)(cs + c0);
            const uint32_t cw[4] = {cv.x, cv.y, cv.z, cv.w};
#pragma unroll
            for (int p = 0; p < 8; ++p) cf[p] = h2f((uint16_t)(cw[p >> 1] >> (16 * (p & 1))));
          } else {
#pragma unroll
            for (int p = 0; p < 8; ++p) cf[p] = 1.f;
          }
          float wv[8];
#pragma unroll
          for (int p = 0; p < 8; ++p) {
            const bool kp = (mb >> p) & 1u;
            wv[p] = kp ? ((float)(win & 0xFu) - z) * cf[p] : 0.f;
            win = kp ? win >> 4 : win;
          }
#pragma unroll
          for (int i = 0; i < M; ++i) {
            const uint4 xv = *(const uint4*)((const uint16_t*)x + (size_t)i * ldx + c0);
            const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
            for (int p = 0; p < 8; ++p) {
              const uint16_t hb = (uint16_t)(xw[p >> 1] >> (16 * (p & 1)));
              part[i] = fmaf(wv[p], XDT == CBK_F16 ? h2f(hb) : bf2f(hb), part[i]);
            }
          }
        }
#pragma unroll
        for (int i = 0; i < M; ++i) acc[i] = fmaf(s, part[i], acc[i]);
      }
    } else {
      const uint8_t* row = m.data + m.row_off[k];
      const uint32_t* bm = (const uint32_t*)row;
      const bool has_goff = false;
      const int hdr = ((m.N >> 3) + 15) & ~15;
      for (int g = lane; g < m.G; g += 64) {
        uint32_t off = 0;
        if (has_goff) off = ((const uint16_t*)(row + (m.N >> 3)))[g];
        else
          for (int gg = 0; gg < g; ++gg) {
            int c = 0;
            for (int i = 0; i < 4; ++i) c += __popc(bm[gg * 4 + i]);
            off += (uint32_t)(c + 1) >> 1;
          }
        const uint8_t* codes = row + hdr + off;
        const float s = h2f(m.scale[(size_t)k * m.G + g]);
        const int z = m.zero[(size_t)k * m.G + g];
        float part[M];
#pragma unroll
        for (int i = 0; i < M; ++i) part[i] = 0.f;
        int nib = 0;
        for (int w4 = 0; w4 < 4; ++w4) {
          uint32_t keep = bm[g * 4 + w4];
          while (keep) {
            const int p = __ffs(keep) - 1;
            keep &= keep - 1;
            const uint32_t by = codes[nib >> 1];
            const int q = (nib & 1) ? (int)(by >> 4) : (int)(by & 0xFu);
            ++nib;
            const int col = g * 128 + w4 * 32 + p;
            const float c = cs ? h2f(cs[col]) : 1.f;
#pragma unroll
            for (int i = 0; i < M; ++i)
              part[i] = fmaf((float)(q - z), load_act<XDT>(x, (size_t)i * ldx + col) * c, part[i]);
          }
        }
#pragma unroll
        for (int i = 0; i < M; ++i) acc[i] = fmaf(s, part[i], acc[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < M; ++i) {
      float v = wave_sum(acc[i]);
      if (lane == 0) {
        if (bias) v += (ydt == CBK_F32) ? ((const float*)bias)[k]
                     : (ydt == CBK_F16) ? h2f(((const uint16_t*)bias)[k]) : bf2f(((const uint16_t*)bias)[k]);
        if (ydt == CBK_F32) ((float*)y)[(size_t)i * ldy + k] = v;
        else if (ydt == CBK_F16) ((uint16_t*)y)[(size_t)i * ldy + k] = f2h(v);
        else ((uint16_t*)y)[(size_t)i * ldy + k] = f2bf(v);
      }
    }
  }
}

template <int XDT, int PATH>
static int launch_p(const DMat& m, const void* x, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                    const void* bias, hipStream_t st) {
  const int blocks = (m.K + 3) / 4 < 4096 ? (m.K + 3) / 4 : 4096;
  const dim3 grid(blocks), blk(256);
  // activation rows are processed in chunks of at most 4 per launch
  for (int m0 = 0; m0 < M; m0 += 4) {
    const int mc = M - m0 < 4 ? M - m0 : 4;
    const void* xs = (const uint8_t*)x + (size_t)m0 * ldx * 2;
    void* ys = (uint8_t*)y + (size_t)m0 * ldy * (ydt == CBK_F32 ? 4 : 2);
    switch (mc) {
      case 1: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 1, PATH>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      case 2: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 2, PATH>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      case 3: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 3, PATH>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      default: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 4, PATH>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
    }
  }
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

template <int XDT>
static int launch_m(const DMat& m, const void* x, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                    const void* bias, hipStream_t st) {
  if (m.layout == CBK_DENSE8) return launch_p<XDT, 0>(m, x, M, ldx, y, ydt, ldy, bias, st);
  if (family_of(m.layout) != FAM_SPARSE) return launch_p<XDT, 1>(m, x, M, ldx, y, ydt, ldy, bias, st);
  if (m.layout != CBK_SPARSE4 || m.G <= SP4_MAX_G) return launch_p<XDT, 2>(m, x, M, ldx, y, ydt, ldy, bias, st);
  return launch_p<XDT, 3>(m, x, M, ldx, y, ydt, ldy, bias, st);
}

int launch_gemv_stream(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*, void*, size_t, hipStream_t);
int launch_gemv_dense8(const DMat&, const void*, int, int, int64_t, void*, int, int64_t, const void*, hipStream_t);

int launch_gemv_generic(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt,
                        int64_t ldy, const void* bias, void* ws, size_t ws_bytes, hipStream_t st) {
  if (family_of(m.layout) == FAM_SPARSE || m.layout == CBK_DENSE8) {   // integer-dot kernels where they apply
    const int rc = m.layout == CBK_DENSE8 ? launch_gemv_dense8(m, x, xdt, M, ldx, y, ydt, ldy, bias, st)
                                          : launch_gemv_stream(m, x, xdt, M, ldx, y, ydt, ldy, bias, ws, ws_bytes, st);
    if (rc != CBK_ERR_UNSUPPORTED) return rc;
  }
  if (xdt == CBK_F16) return launch_m<CBK_F16>(m, x, M, ldx, y, ydt, ldy, bias, st);
  if (xdt == CBK_BF16T) return launch_m<CBK_BF16T>(m, x, M, ldx, y, ydt, ldy, bias, st);
  return CBK_ERR_DTYPE;
}

}  // namespace cbk
