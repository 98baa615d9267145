// Packed bytes -> dense W_hat, bit-exact float32 evaluation of
//   ((q - zero) * scale) * keep * col_scale
// in that order (reference: src/cobaltkernel/dequant_ref.py:69-82), then one RN-even cast.
// One thread owns one (row, 32-column block); a block of 32 columns never crosses a
// quantisation group because the group is 64 or 128.
#include "cbk_device.h"

namespace cbk {

template <int ODT>
__global__ __launch_bounds__(256) void dequant_fixed_kernel(DMat m, int row0, int nrows, int with_cs,
                                                            void* out, int64_t ld) {
  const int NB = m.N / BLOCK;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)nrows * NB) return;
  const int r = (int)(gid / NB), t = (int)(gid % NB);
  const int k = row0 + r;
  const RowView row = row_view(m, k);
  int q[32];
  const uint32_t keep = decode_block32(m, row, t, q);
  const int g = (t * BLOCK) / m.group;
  const float s = h2f(m.scale[meta_index(m, k, g)]);
  const float z = (float)m.zero[meta_index(m, k, g)];
  const uint16_t* cs = (with_cs && m.cs) ? m.cs + (size_t)cs_row_of(m, k) * m.N + t * BLOCK : nullptr;
  const bool dense = family_of(m.layout) == FAM_DENSE;
#pragma unroll
  for (int p = 0; p < 32; ++p) {
    float w = __fmul_rn((float)q[p] - z, s);
    if (!dense) w = __fmul_rn(w, (float)((keep >> p) & 1u));
    if (cs) w = __fmul_rn(w, h2f(cs[p]));
    store_out<ODT>(out, (size_t)r * ld + t * BLOCK + p, w);
  }
}

// SPARSE4 / SPARSE4X / SPARSE4E (src/cobaltkernel/pack_cobalt.py:201-250): per row
// [bitmap N/8][uint16 goff[G] padded to 16 B, 4X/4E only][pad to 16][nibbles]; group g's
// survivor nibbles start at byte goff[g], each group padded to an even nibble count.
template <int ODT>
__global__ __launch_bounds__(256) void dequant_sparse_kernel(DMat m, int row0, int nrows, int with_cs,
                                                             void* out, int64_t ld) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)nrows * m.G) return;
  const int r = (int)(gid / m.G), g = (int)(gid % m.G);
  const int k = row0 + r;
  const uint8_t* row = m.data + m.row_off[k];
  const uint32_t* bm = (const uint32_t*)row;
  const bool has_goff = m.layout != CBK_SPARSE4;
  const int hdr = ((m.N >> 3) + (has_goff ? ((m.G * 2 + 15) & ~15) : 0) + 15) & ~15;
  uint32_t off;
  if (has_goff) {
    off = ((const uint16_t*)(row + (m.N >> 3)))[g];
  } else {
    off = 0;
    for (int gg = 0; gg < g; ++gg) {
      int c = 0;
      for (int i = 0; i < 4; ++i) c += __popc(bm[gg * 4 + i]);
      off += (uint32_t)(c + 1) >> 1;
    }
  }
  const uint8_t* codes = row + hdr + off;
  const float s = h2f(m.scale[(size_t)k * m.G + g]);
  const float z = (float)m.zero[(size_t)k * m.G + g];
  const uint16_t* cs = (with_cs && m.cs) ? m.cs + (size_t)cs_row_of(m, k) * m.N + g * 128 : nullptr;
  int nib = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t keep = bm[g * 4 + i];
    for (int p = 0; p < 32; ++p) {
      float w = 0.0f;
      if ((keep >> p) & 1u) {
        const uint32_t by = codes[nib >> 1];
        const int q = (nib & 1) ? (int)(by >> 4) : (int)(by & 0xFu);
        ++nib;
        w = __fmul_rn((float)q - z, s);
        if (cs) w = __fmul_rn(w, h2f(cs[i * 32 + p]));
      }
      store_out<ODT>(out, (size_t)r * ld + g * 128 + i * 32 + p, w);
    }
  }
}

int launch_dequant(const DMat& m, int row0, int nrows, int with_cs, void* out, int odt, int64_t ld,
                   hipStream_t st) {
  if (nrows == 0) return CBK_OK;
  const bool sparse = family_of(m.layout) == FAM_SPARSE;
  const int64_t items = (int64_t)nrows * (sparse ? m.G : m.N / BLOCK);
  const dim3 grid((unsigned)((items + 255) / 256)), blk(256);
#define CBK_LAUNCH(ODT)                                                                     \
  do {                                                                                      \
    if (sparse) hipLaunchKernelGGL(dequant_sparse_kernel<ODT>, grid, blk, 0, st, m, row0,   \
                                   nrows, with_cs, out, ld);                                \
    else hipLaunchKernelGGL(dequant_fixed_kernel<ODT>, grid, blk, 0, st, m, row0, nrows,    \
                            with_cs, out, ld);                                              \
  } while (0)
  if (odt == CBK_F32) CBK_LAUNCH(CBK_F32);
  else if (odt == CBK_F16) CBK_LAUNCH(CBK_F16);
  else if (odt == CBK_BF16T) CBK_LAUNCH(CBK_BF16T);
  else return CBK_ERR_DTYPE;
#undef CBK_LAUNCH
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

}  // namespace cbk
