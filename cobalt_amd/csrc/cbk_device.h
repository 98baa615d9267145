// Device-side view of a CBK1 packed matrix and the bit-level readers every kernel shares.
// gfx950 only.  Byte layouts follow docs/FORMAT.md:83-122 of the reference for layouts 0-7;
// layouts 8 (BLKC) and 9 (DENSEB) are one LSB-first bit stream per row (see include/cbk.h).
//
// Two byte orders of the same rows are read: the reference's row-major order, and the
// 16-row tile-interleaved order (CBK_FLAG_TILED16) in which 16-byte unit u of row k sits at
// (k/16)*16*stride + (u*16 + k%16)*16, so that the sixteen rows a wavefront decodes
// together are one contiguous run in HBM.  Kernels address rows only through RowView.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include "../../include/cbk.h"

namespace cbk {

constexpr int BLOCK = 32;          // mask block: 32 input columns, one uint32 of the bitmap

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// What a kernel receives by value.  Built on the host from a checked cbk_desc.
struct DMat {
  const uint8_t* data;
  const uint32_t* row_off;
  const uint16_t* scale;     // fp16 bits
  const uint8_t* zero;
  const uint16_t* cs;        // fp16 bits, [cs_rows, N] or nullptr
  int K, N, G;
  int layout, bits, group, keep;
  int cs_rows, cs_split0, cs_split1;
  int flags;
  int tiled;                 // 1: 16-row tile-interleaved byte order
  uint32_t stride;           // bytes per row (fixed-stride layouts)
  uint32_t code_off;         // byte offset of the code plane inside a row
};

enum Family { FAM_DENSE = 0, FAM_BLK = 1, FAM_BLK6 = 2, FAM_SPARSE = 3 };

__host__ __device__ inline int family_of(int layout) {
  switch (layout) {
    case CBK_DENSE4: case CBK_DENSE8: case CBK_DENSEB: return FAM_DENSE;
    case CBK_BLK1632_4: case CBK_BLKC: return FAM_BLK;
    case CBK_BLK1632_6: return FAM_BLK6;
    default: return FAM_SPARSE;
  }
}

// One row of a fixed-stride matrix in either byte order: unit(u) is the address of its
// 16-byte unit u, dword(d) its d-th little-endian dword.
struct RowView {
  const uint8_t* base;
  uint32_t ustride;          // bytes from one 16-byte unit of the row to the next
  __device__ inline const uint8_t* unit(uint32_t u) const { return base + (size_t)u * ustride; }
  __device__ inline uint32_t dword(uint32_t d) const {
    return *(const uint32_t*)(base + (size_t)(d >> 2) * ustride + (d & 3u) * 4u);
  }
};
__device__ inline RowView row_view(const DMat& m, int k) {
  RowView r;
  if (m.tiled) { r.base = m.data + (size_t)(k >> 4) * m.stride * 16 + (size_t)(k & 15) * 16; r.ustride = 256; }
  else { r.base = m.data + (size_t)k * m.stride; r.ustride = 16; }
  return r;
}
// index of the scale / zero entry of (row k, group g)
__device__ inline size_t meta_index(const DMat& m, int k, int g) {
  return m.tiled ? ((size_t)(k >> 4) * m.G + g) * 16 + (k & 15) : (size_t)k * m.G + g;
}

// ------------------------------------------------------------------ scalar conversions
__device__ inline float h2f(uint16_t h) {            // exact, subnormals included
  return __half2float(__ushort_as_half(h));
}
__device__ inline float bf2f(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ inline uint16_t f2bf(float f) {            // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ inline uint16_t f2h(float f) { return __half_as_ushort(__float2half_rn(f)); }
// The power of two s >= 1 with mx / s in [2^14, 2^15) for a finite mx >= 2^15, else 1 (the
// exponent arithmetic holds for every finite float; an infinite or NaN maximum is left alone).  The GEMM
// kernels feed the fp16 matrix pipe: a token whose activations reach beyond fp16's range is
// divided by s before the cast and its outputs are multiplied by s, both exact.
__device__ inline float token_scale(float mx) {
  if (!(mx >= 32768.f) || !(mx <= 3.4028234663852886e38f)) return 1.f;
  const uint32_t e = ((__float_as_uint(mx) >> 23) & 0xffu) - 14u;      // biased exponent of mx, less 14
  return __uint_as_float(e << 23);
}

template <int DT> __device__ inline float load_act(const void* p, size_t i) {
  if (DT == CBK_F16) return h2f(((const uint16_t*)p)[i]);
  if (DT == CBK_BF16T) return bf2f(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}
template <int DT> __device__ inline void store_out(void* p, size_t i, float v) {
  if (DT == CBK_F16) ((uint16_t*)p)[i] = f2h(v);
  else if (DT == CBK_BF16T) ((uint16_t*)p)[i] = f2bf(v);
  else ((float*)p)[i] = v;
}

__device__ inline int cs_row_of(const DMat& m, int k) {
  if (m.cs_rows <= 1) return 0;
  if (m.cs_rows == 2) return k & 1;
  return k < m.cs_split0 ? 0 : (k < m.cs_split0 + m.cs_split1 ? 1 : 2);
}

// ------------------------------------------------------------------ generic 32-column reader
// Codes of the 32 columns of block t of a row (fixed-stride layouts).  q[p] is the stored code
// for a kept column and 0 for a pruned one; the return value is the keep bitmap (all ones for
// the dense family, whose pruned columns hold the zero point).  Everything is indexed with
// compile-time constants after unrolling, so q[] stays in VGPRs.
__device__ inline uint32_t decode_block32(const DMat& m, const RowView& row, int t, int (&q)[32]) {
  const int fam = family_of(m.layout);
  const int b = m.bits;
  const uint32_t cm = (1u << b) - 1u;
  if (fam == FAM_DENSE) {
    // 32 codes = b dwords, dword aligned; code p at bits [p*b, p*b+b)
    const uint32_t d0 = (uint32_t)t * b;
    uint64_t cur = 0; int have = 0, wi = 0;
#pragma unroll
    for (int p = 0; p < 32; ++p) {
      if (have < b) { cur |= ((uint64_t)row.dword(d0 + wi++)) << have; have += 32; }
      q[p] = (int)((uint32_t)cur & cm);
      cur >>= b; have -= b;
    }
    return 0xffffffffu;
  }
  const uint32_t keep = row.dword(t);
  if (fam == FAM_BLK6) {
    const uint32_t nd = (uint32_t)(m.N >> 5);              // dwords of the mask plane
    uint64_t lo = (uint64_t)row.dword(nd + 2 * t) | ((uint64_t)row.dword(nd + 2 * t + 1) << 32);
    const uint32_t hw = row.dword(3 * nd + t);
    uint32_t he = hw & 0xffffu, ho = hw >> 16;
    int i = 0;
#pragma unroll
    for (int p = 0; p < 32; ++p) {
      const bool kp = (keep >> p) & 1u;
      uint32_t hi = (i & 1) ? (ho & 3u) : (he & 3u);
      q[p] = kp ? (int)(((uint32_t)lo & 0xFu) | (hi << 4)) : 0;
      if (kp) { lo >>= 4; if (i & 1) ho >>= 2; else he >>= 2; ++i; }
    }
    return keep;
  }
  // FAM_BLK: survivor i of block t at bits [(t*keep+i)*b, ...) of the code plane
  const uint32_t sb = (uint32_t)t * (uint32_t)(m.keep * b);
  const uint32_t d0 = (m.code_off >> 2) + (sb >> 5);
  const uint32_t sh = sb & 31u;
  uint32_t e[5];
#pragma unroll
  for (int i = 0; i < 5; ++i) e[i] = row.dword(d0 + i);    // <= 128 code bits + 31 bits of skew
  uint64_t lo = ((uint64_t)__builtin_amdgcn_alignbit(e[1], e[0], sh)) |
                ((uint64_t)__builtin_amdgcn_alignbit(e[2], e[1], sh) << 32);
  uint64_t hi = ((uint64_t)__builtin_amdgcn_alignbit(e[3], e[2], sh)) |
                ((uint64_t)__builtin_amdgcn_alignbit(e[4], e[3], sh) << 32);
#pragma unroll
  for (int p = 0; p < 32; ++p) {
    const bool kp = (keep >> p) & 1u;
    q[p] = kp ? (int)((uint32_t)lo & cm) : 0;
    if (kp) { lo = (lo >> b) | (hi << (64 - b)); hi >>= b; }
  }
  return keep;
}

}  // namespace cbk
