// Reference-shaped decode GEMV for EVERY layout: one wavefront per weight row, lanes stride
// over 32-column blocks, float32 FMA, butterfly reduction.  It is the path for layouts and
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

template <int XDT, int M>
__global__ __launch_bounds__(256) void gemv_generic_kernel(DMat m, const void* x, int64_t ldx, void* y,
                                                           int ydt, int64_t ldy, const void* bias) {
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int nwaves = (gridDim.x * blockDim.x) >> 6;
  const int fam = family_of(m.layout);
  for (int k = wave; k < m.K; k += nwaves) {
    float acc[M];
#pragma unroll
    for (int i = 0; i < M; ++i) acc[i] = 0.f;
    const uint16_t* cs = m.cs ? m.cs + (size_t)cs_row_of(m, k) * m.N : nullptr;
    if (fam != FAM_SPARSE) {
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
    } else {
      const uint8_t* row = m.data + m.row_off[k];
      const uint32_t* bm = (const uint32_t*)row;
      const bool has_goff = m.layout != CBK_SPARSE4;
      const int hdr = ((m.N >> 3) + (has_goff ? ((m.G * 2 + 15) & ~15) : 0) + 15) & ~15;
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

template <int XDT>
static int launch_m(const DMat& m, const void* x, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                    const void* bias, hipStream_t st) {
  const int blocks = (m.K + 3) / 4 < 4096 ? (m.K + 3) / 4 : 4096;
  const dim3 grid(blocks), blk(256);
  // activation rows are processed in chunks of at most 4 per launch
  for (int m0 = 0; m0 < M; m0 += 4) {
    const int mc = M - m0 < 4 ? M - m0 : 4;
    const void* xs = (const uint8_t*)x + (size_t)m0 * ldx * 2;
    void* ys = (uint8_t*)y + (size_t)m0 * ldy * (ydt == CBK_F32 ? 4 : 2);
    switch (mc) {
      case 1: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 1>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      case 2: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 2>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      case 3: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 3>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
      default: hipLaunchKernelGGL((gemv_generic_kernel<XDT, 4>), grid, blk, 0, st, m, xs, ldx, ys, ydt, ldy, bias); break;
    }
  }
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

int launch_gemv_generic(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt,
                        int64_t ldy, const void* bias, hipStream_t st) {
  if (xdt == CBK_F16) return launch_m<CBK_F16>(m, x, M, ldx, y, ydt, ldy, bias, st);
  if (xdt == CBK_BF16T) return launch_m<CBK_BF16T>(m, x, M, ldx, y, ydt, ldy, bias, st);
  return CBK_ERR_DTYPE;
}

}  // namespace cbk
