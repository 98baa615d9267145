// RAW arrays (bitmap, codes, scale, zero point) -> the byte image the kernels read, on the GPU.
// The byte layouts are those of the reference's packer (src/cobaltkernel/pack_cobalt.py:98-250,
// docs/FORMAT.md:83-122) and of the two bit-stream layouts of this library (include/cbk.h);
// the destination is either the row-major order or the 16-row tiled order.
//
// One thread packs 256 columns of one row (128 at the end of a row whose length is an odd
// multiple of 128): 8 mask blocks, whose code bits end on a byte boundary whatever the code
// width and the survivors per block, so no two threads share a byte.  HBM-bound byte work:
// it reads K*N code bytes and K*N/8 mask bytes and writes the packed rows once.
#include "cbk_device.h"

namespace cbk {

struct PackArgs {
  const uint8_t* mask;     // [K, N/8] or nullptr
  const uint8_t* q;        // [K, N]
  const uint16_t* scale;   // fp16 [K, G]
  const void* zero;        // fp16 or uint8 [K, G]
  uint8_t* data;
  uint16_t* oscale;
  uint8_t* ozero;
  int K, N, G, group, bits, keep, fam, tiled, zero_f16, fix_zero;
  uint32_t stride;
};

__device__ inline uint8_t* dst_byte(const PackArgs& a, int k, uint32_t o) {
  if (a.tiled) return a.data + (size_t)(k >> 4) * 16 * a.stride + ((size_t)(o >> 4) * 16 + (k & 15)) * 16 + (o & 15);
  return a.data + (size_t)k * a.stride + o;
}

// LSB-first bit stream writer onto consecutive row bytes starting at byte `o`
struct BitSink {
  uint64_t acc = 0;
  int n = 0;
  uint32_t o;
  __device__ inline void put(const PackArgs& a, int k, uint32_t code, int bits) {
    acc |= (uint64_t)(code & ((1u << bits) - 1u)) << n;            // never into the neighbouring code
    n += bits;
    while (n >= 8) { *dst_byte(a, k, o++) = (uint8_t)acc; acc >>= 8; n -= 8; }
  }
  __device__ inline void flush(const PackArgs& a, int k) {
    if (n > 0) { *dst_byte(a, k, o++) = (uint8_t)acc; acc = 0; n = 0; }
  }
};

// The quantisation of one group as it is stored: the RAW one, or, when the RAW zero point is off
// the code grid [0, 2^bits - 1], one re-derived from the hull of the group's dequantised
// survivors and 0 (src/cobaltkernel/pack_cobalt.py:55-87).  Every step is a single correctly
// rounded float32 operation in the reference's order, so the bytes do not depend on the device.
struct GroupQ {
  bool redo;
  float z_raw, s_raw, s_new, z_new;
  uint32_t z_out;
  uint16_t s_out;
  __device__ inline uint32_t code(uint32_t q, float nl) const {
    if (!redo) return q > (uint32_t)nl ? (uint32_t)nl : q;
    const float v = __fmul_rn((float)q - z_raw, s_raw);
    return (uint32_t)fminf(fmaxf(rintf(__fadd_rn(__fdiv_rn(v, s_new), z_new)), 0.f), nl);
  }
};

__device__ inline GroupQ group_quant(const PackArgs& a, int k, int g, const uint8_t* qrow_full, const uint8_t* mrow_full) {
  GroupQ r;
  const size_t gi = (size_t)k * a.G + g;
  const float nl = (float)((1u << a.bits) - 1u);
  r.s_out = a.scale[gi];
  r.s_raw = h2f(r.s_out);
  int zi;
  if (a.zero_f16) zi = (int)rintf(h2f(((const uint16_t*)a.zero)[gi]));
  else zi = (int)((const uint8_t*)a.zero)[gi];
  r.z_raw = (float)zi;
  r.redo = a.fix_zero && (zi < 0 || zi > (int)nl);
  r.z_out = (uint32_t)zi & 0xffu;
  r.s_new = r.s_raw; r.z_new = r.z_raw;
  if (!r.redo) return r;
  float vmin = 3.4028234663852886e38f, vmax = -3.4028234663852886e38f;
  bool any = false;
  for (int j = g * a.group; j < (g + 1) * a.group; ++j) {
    const bool kept = mrow_full ? ((mrow_full[j >> 3] >> (j & 7)) & 1u) != 0 : true;
    if (!kept) continue;
    const float v = __fmul_rn((float)qrow_full[j] - r.z_raw, r.s_raw);
    vmin = fminf(vmin, v); vmax = fmaxf(vmax, v); any = true;
  }
  if (!any) vmin = vmax = 0.f;
  vmin = fminf(vmin, 0.f); vmax = fmaxf(vmax, 0.f);
  r.s_new = fmaxf(__fdiv_rn(__fsub_rn(vmax, vmin), nl), 1e-12f);
  r.z_new = fminf(fmaxf(rintf(__fdiv_rn(-vmin, r.s_new)), 0.f), nl);
  r.z_out = (uint32_t)r.z_new;
  r.s_out = f2h(r.s_new);
  return r;
}

// status[0] |= 1: a block without exactly `keep` survivors; |= 2: a dense layout had to store a zero
// point above 2^bits - 1 at a pruned column (its low bits are stored; the column no longer
// dequantises to 0); status[1] += groups re-derived
__global__ __launch_bounds__(256) void pack_rows_kernel(PackArgs a, int* status) {
  const int units = (a.N + 255) >> 8;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)a.K * units) return;
  const int k = (int)(id / units), u = (int)(id % units);
  const int c0 = u << 8, nb = (a.N - c0 >= 256 ? 256 : a.N - c0) >> 5;     // 8 or 4 blocks
  const uint8_t* qfull = a.q + (size_t)k * a.N;
  const uint8_t* mfull = a.mask ? a.mask + (size_t)k * (a.N >> 3) : nullptr;
  const uint8_t* qrow = qfull + c0;
  const uint8_t* mrow = mfull ? mfull + (c0 >> 3) : nullptr;
  const float nl = (float)((1u << a.bits) - 1u);
  BitSink sink;
  if (a.fam == FAM_DENSE) sink.o = (uint32_t)(c0 >> 3) * a.bits;
  else sink.o = (uint32_t)(a.N >> 3) + (uint32_t)(c0 >> 5) * a.keep * a.bits / 8;   // c0/32 is a multiple of 8
  bool wrong = false, off_grid = false;
  int fixed = 0, g_now = -1;
  GroupQ gq;
  for (int t = 0; t < nb; ++t) {
    const int g = (c0 + 32 * t) / a.group;
    if (g != g_now) {                                              // groups are 64 or 128 columns: never across units
      g_now = g;
      gq = group_quant(a, k, g, qfull, mfull);
      fixed += gq.redo ? 1 : 0;
      const size_t mi = a.tiled ? ((size_t)(k >> 4) * a.G + g) * 16 + (k & 15) : (size_t)k * a.G + g;
      a.oscale[mi] = gq.s_out;
      a.ozero[mi] = (uint8_t)gq.z_out;
    }
    const uint32_t m = mrow ? *(const uint32_t*)(mrow + 4 * t) : 0xffffffffu;
    __attribute__((aligned(16))) uint8_t c[32];
    *(uint4*)(c) = *(const uint4*)(qrow + 32 * t);
    *(uint4*)(c + 16) = *(const uint4*)(qrow + 32 * t + 16);
    if (a.fam == FAM_DENSE) {
      if (m != 0xffffffffu && gq.z_out > (uint32_t)nl) off_grid = true;
#pragma unroll
      for (int j = 0; j < 32; ++j) sink.put(a, k, ((m >> j) & 1u) ? gq.code(c[j], nl) : gq.z_out, a.bits);
      continue;
    }
    const uint32_t blk = (uint32_t)(c0 >> 5) + t;
#pragma unroll
    for (int i = 0; i < 4; ++i) *dst_byte(a, k, blk * 4 + i) = (uint8_t)(m >> (8 * i));
    if (__popc(m) != a.keep) wrong = true;
    if (a.fam == FAM_BLK6) {                                       // low nibbles, then 2 high bits: even survivors in
      uint32_t lo[2] = {0, 0}, hw = 0;                             // the low half of the word, odd ones in the high half
      int i = 0;
#pragma unroll
      for (int j = 0; j < 32; ++j)
        if (((m >> j) & 1u) && i < 16) {
          const uint32_t cd = gq.code(c[j], nl);
          lo[i >> 3] |= (cd & 0xF) << (4 * (i & 7));
          hw |= ((cd >> 4) & 3) << (2 * (i >> 1) + 16 * (i & 1));
          ++i;
        }
#pragma unroll
      for (int b = 0; b < 8; ++b) *dst_byte(a, k, (uint32_t)(a.N >> 3) + blk * 8 + b) = (uint8_t)(lo[b >> 2] >> (8 * (b & 3)));
#pragma unroll
      for (int b = 0; b < 4; ++b) *dst_byte(a, k, (uint32_t)(a.N * 3 >> 3) + blk * 4 + b) = (uint8_t)(hw >> (8 * b));
    } else {
      int i = 0;
#pragma unroll
      for (int j = 0; j < 32; ++j)
        if (((m >> j) & 1u) && i < a.keep) { sink.put(a, k, gq.code(c[j], nl), a.bits); ++i; }
      for (; i < a.keep; ++i) sink.put(a, k, 0, a.bits);           // too few survivors: keep the stream aligned
    }
  }
  sink.flush(a, k);
  if (status) {
    if (wrong) atomicOr(status, 1);
    if (off_grid) atomicOr(status, 2);
    if (fixed) atomicAdd(status + 1, fixed);
  }
}

__global__ __launch_bounds__(256) void pack_clear_kernel(uint4* p, size_t n16) {
  const size_t id = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (id < n16) p[id] = make_uint4(0, 0, 0, 0);
}

static void clear16(void* p, size_t bytes, hipStream_t st) {
  hipLaunchKernelGGL(pack_clear_kernel, dim3((unsigned)((bytes / 16 + 255) / 256)), dim3(256), 0, st, (uint4*)p, bytes / 16);
}

// ------------------------------------------------------------------ the way back: image -> RAW
// Codes (0 at a pruned column of a bitmap or survivor-stream layout, the stored code, i.e. the
// zero point, at a pruned column of a dense layout) and the keep bitmap of any layout.
// Fixed-stride layouts: one thread per (row, 32-column block); survivor streams: one thread
// per (row, group), as in the dequantiser.
__global__ __launch_bounds__(256) void unpack_fixed_kernel(DMat m, uint8_t* q, uint8_t* mask) {
  const int NB = m.N / BLOCK;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)m.K * NB) return;
  const int k = (int)(gid / NB), t = (int)(gid % NB);
  int c[32];
  const uint32_t keep = decode_block32(m, row_view(m, k), t, c);
  uint32_t w[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    w[i] = (uint32_t)c[4 * i] | ((uint32_t)c[4 * i + 1] << 8) | ((uint32_t)c[4 * i + 2] << 16) | ((uint32_t)c[4 * i + 3] << 24);
  uint4* dst = (uint4*)(q + (size_t)k * m.N + t * BLOCK);
  dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
  dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
  if (mask) *(uint32_t*)(mask + (size_t)k * (m.N >> 3) + t * 4) = keep;
}

__global__ __launch_bounds__(256) void unpack_sparse_kernel(DMat m, uint8_t* q, uint8_t* mask) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)m.K * m.G) return;
  const int k = (int)(gid / m.G), g = (int)(gid % m.G);
  const uint8_t* row = m.data + m.row_off[k];
  const uint32_t* bm = (const uint32_t*)row;
  const bool has_goff = m.layout != CBK_SPARSE4;
  const int hdr = ((m.N >> 3) + (has_goff ? ((m.G * 2 + 15) & ~15) : 0) + 15) & ~15;
  uint32_t off = 0;
  if (has_goff) {
    off = ((const uint16_t*)(row + (m.N >> 3)))[g];
  } else {
    for (int gg = 0; gg < g; ++gg) {
      int c = 0;
      for (int i = 0; i < 4; ++i) c += __popc(bm[gg * 4 + i]);
      off += (uint32_t)(c + 1) >> 1;
    }
  }
  const uint8_t* codes = row + hdr + off;
  int nib = 0;
  for (int i = 0; i < 4; ++i) {
    const uint32_t keep = bm[g * 4 + i];
    uint32_t w[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = 0;
#pragma unroll
    for (int p = 0; p < 32; ++p) {
      if ((keep >> p) & 1u) {
        const uint32_t by = codes[nib >> 1];
        const uint32_t c = (nib & 1) ? (by >> 4) : (by & 0xFu);
        ++nib;
        w[p >> 2] |= c << (8 * (p & 3));
      }
    }
    uint4* dst = (uint4*)(q + (size_t)k * m.N + g * 128 + i * 32);
    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
    if (mask) *(uint32_t*)(mask + (size_t)k * (m.N >> 3) + g * 16 + i * 4) = keep;
  }
}

int launch_unpack(const DMat& m, void* q, void* mask, hipStream_t st) {
  const bool sparse = family_of(m.layout) == FAM_SPARSE;
  const int64_t items = (int64_t)m.K * (sparse ? m.G : m.N / BLOCK);
  const dim3 grid((unsigned)((items + 255) / 256)), blk(256);
  if (sparse) hipLaunchKernelGGL(unpack_sparse_kernel, grid, blk, 0, st, m, (uint8_t*)q, (uint8_t*)mask);
  else hipLaunchKernelGGL(unpack_fixed_kernel, grid, blk, 0, st, m, (uint8_t*)q, (uint8_t*)mask);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

int launch_pack(const DMat& m, const void* mask, const void* q, const void* scale, const void* zero, int zero_f16,
                int fix_zero, int* status, hipStream_t st) {
  const int fam = family_of(m.layout);
  if (fam == FAM_SPARSE) return CBK_ERR_UNSUPPORTED;
  const int kr = m.tiled ? (m.K + 15) / 16 * 16 : m.K;
  clear16((void*)m.data, (size_t)kr * m.stride + (m.tiled ? 512 : 64), st);      // rows + tail, a multiple of 16
  if (m.tiled && kr != m.K) {                                      // entries of the padding rows
    clear16((void*)m.scale, (size_t)kr * m.G * 2, st);
    clear16((void*)m.zero, (size_t)kr * m.G, st);
  }
  PackArgs a;
  a.mask = (const uint8_t*)mask; a.q = (const uint8_t*)q; a.scale = (const uint16_t*)scale; a.zero = zero;
  a.data = (uint8_t*)m.data; a.oscale = (uint16_t*)m.scale; a.ozero = (uint8_t*)m.zero;
  a.K = m.K; a.N = m.N; a.G = m.G; a.group = m.group; a.bits = m.bits; a.keep = m.keep; a.fam = fam; a.tiled = m.tiled;
  a.zero_f16 = zero_f16; a.fix_zero = fix_zero;
  a.stride = m.stride;
  const int64_t items = (int64_t)m.K * ((m.N + 255) / 256);
  hipLaunchKernelGGL(pack_rows_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, a, status);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

}  // namespace cbk
