// Bit-level decoding shared by the decode GEMV and the prefill GEMM: the byte-permute
// expansion of a pruning bitmap (selector table, code-stream windows, 3-bit widening) and the
// compile-time description of a (bits, keep, group) configuration.  gfx950 only.
#pragma once
#include "cbk_device.h"

namespace cbk {

// ------------------------------------------------------------------ selector table
// Entry for mask byte mb: eight v_perm_b32 selector bytes, one per column.  A kept column
// with r survivors before it in the byte selects pool byte idx(r); a pruned column selects
// 0x0C, the constant 0x00.
// kind 0: pool = {even-rank codes (bytes 0-3), odd-rank codes (bytes 4-7)}   (4-bit codes)
// kind 1: pool = {c0,c4,c1,c5 | c2,c6,c3,c7}                                   (2-bit codes)
__device__ inline uint2 make_selectors(uint32_t mb, int kind) {
  uint32_t lo = 0, hi = 0, r = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const uint32_t idx = kind == 0 ? ((r >> 1) + 4u * (r & 1u)) : (((r & 3u) << 1) | (r >> 2));
    const bool kp = (mb >> p) & 1u;
    const uint32_t sel = kp ? idx : 0x0Cu;
    if (p < 4) lo |= sel << (8 * p); else hi |= sel << (8 * (p - 4));
    r += kp ? 1u : 0u;
  }
  return make_uint2(lo, hi);
}

// ------------------------------------------------------------------ small helpers
__device__ inline uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);   // bytes 0-3 of the pool = lo, 4-7 = hi
}

// 32 bits starting at compile-time bit position `pos` of a little-endian dword array
template <int ND>
__device__ inline uint32_t get32(const uint32_t (&w)[ND], int pos) {
  const int i = pos >> 5, s = pos & 31;
  const uint32_t lo = i < ND ? w[i] : 0u, hi = (i + 1) < ND ? w[i + 1] : 0u;
  return s ? __builtin_amdgcn_alignbit(hi, lo, s) : lo;
}

// eight 3-bit codes (24 bits) -> eight nibbles
__device__ inline uint32_t expand3to4(uint32_t w) {
  uint32_t x = (w & 0xFFFu) | ((w & 0xFFF000u) << 4);
  x = (x & 0x003F003Fu) | ((x & 0x0FC00FC0u) << 2);
  x = (x & 0x07070707u) | ((x & 0x38383838u) << 1);
  return x;
}

// 32 bits at a run-time (per-lane) bit offset of an NW-dword stream
template <int NW>
__device__ inline uint32_t window(const uint32_t (&s)[NW], uint32_t sh) {
  // sh can reach 32*NW when every survivor of the block lies before this mask byte; the
  // result is then unused (no selector points into the pool), but the shift must stay defined
  if (NW == 1) return s[0] >> (sh & 31u);
  if (NW == 2) return (uint32_t)((((uint64_t)s[1] << 32) | s[0]) >> (sh & 63u));
  const uint32_t idx = sh >> 5;
  uint32_t w = __builtin_amdgcn_alignbit(s[1], s[0], sh);
#pragma unroll
  for (int i = 1; i < NW; ++i) {
    const uint32_t hi = (i + 1) < NW ? s[i + 1] : 0u;
    const uint32_t c = __builtin_amdgcn_alignbit(hi, s[i], sh);
    w = idx == (uint32_t)i ? c : w;
  }
  return w;
}

// Bitwise select under an all-ones / all-zeros mask (see align_chunk_codes for why not `c ? b : a`).
__device__ inline uint32_t mask_select(uint32_t mask, uint32_t if_clear, uint32_t if_set) {
  return (if_set & mask) | (if_clear & ~mask);                   // one v_bfi_b32
}

// BLK1632_6: the high two bits of the eight survivors from rank r on, as the two byte pools of
// decode (even positions of the window, odd positions), already at bits 4-5 of their bytes.
// Survivor i of a block keeps its high bits at bit i of the block's dword if i is even, at bit
// i + 15 if it is odd (src/cobaltkernel/dequant_ref.py:61-66).
__device__ inline uint32_t spread_hi2(uint32_t f) {               // four 2-bit fields -> bits 4-5 of four bytes
  uint32_t x = f & 0xFFu;
  x = (x | (x << 12)) & 0x000F000Fu;
  x = (x | (x << 6)) & 0x03030303u;
  return x << 4;
}
__device__ inline void hi2_pools(uint32_t hw, uint32_t r, uint32_t& h0, uint32_t& h1) {
  const uint32_t odd = r & 1u;
  h0 = spread_hi2(hw >> ((r + 15u * odd) & 31u));                 // positions r, r+2, r+4, r+6
  h1 = spread_hi2(hw >> ((r + 16u - 15u * odd) & 31u));           // positions r+1, r+3, r+5, r+7
}

// pool bytes holding a code q each  ->  signed bytes q - z   (z <= 128, carried in nz)
__device__ inline uint32_t bias_pool(uint32_t codes, uint32_t nz) { return (codes + nz) ^ 0x80808080u; }

// ------------------------------------------------------------------ code-stream configuration
// BITS: code width.  KEEP: survivors per 32 columns, 0 = dense family.  GRP: group size.
template <int BITS, int KEEP, int GRP>
struct CodeCfg {
  static constexpr bool DENSE = KEEP == 0;
  // BITS 6 is BLK1632_6: a 4-bit stream of low nibbles exactly like BLK1632_4, and the two high
  // bits of every survivor in a plane of their own (one dword per block)
  static constexpr bool HI2 = BITS == 6;
  static constexpr int PB = HI2 ? 4 : BITS;                       // bits per code in the stream plane
  static constexpr int CB = DENSE ? 32 * PB : KEEP * PB;          // code bits per 32-column block
  static constexpr int CHB = 4 * CB;                              // per 128-column chunk
  static constexpr bool ALIGNED = CHB % 32 == 0;
  static constexpr int ND = (CHB + 31) / 32;                      // dwords of chunk code bits
  static constexpr bool VEC16 = CHB % 128 == 0;                   // chunks start on 16-byte units
  static constexpr int NL = VEC16 ? ND : 4 * ((CHB + 254) / 128); // dwords loaded: whole units covering any skew
  static constexpr int NIB = DENSE ? 32 : KEEP;                   // codes per block
  static constexpr int SB = BITS == 3 ? 4 : PB;                   // stream code width after expansion
  static constexpr int NW = (NIB * SB + 31) / 32;                 // dwords of a block's code stream
  static constexpr int NGC = 128 / GRP;                           // groups per chunk (1 or 2)
  static constexpr int SEL_KIND = (BITS == 2) ? 1 : 0;
};

// Chunk code bits with their first bit at bit 0 of cw[0], from the NL dwords loaded as whole
// 16-byte units around them; `chunk` is the chunk index the units were loaded for.
template <class C>
__device__ inline void align_chunk_codes(const uint32_t (&raw)[C::NL], uint32_t chunk, uint32_t (&cw)[C::ND]) {
  if (C::VEC16) {
#pragma unroll
    for (int i = 0; i < C::ND; ++i) cw[i] = raw[i];
  } else {
    const uint32_t skew = (chunk * C::CHB) & 127u;                // inside the first unit
    uint32_t t1[C::NL];
#pragma unroll
    for (int i = 0; i < C::NL; ++i)
      t1[i] = C::ALIGNED ? raw[i] : __builtin_amdgcn_alignbit(i + 1 < C::NL ? raw[i + 1] : 0u, raw[i], skew);
    // Shift by one and by two dwords with bitwise selects under a sign-extended bit of the skew.
    // Written as C++ conditionals the compiler turns the two steps into one read of the array at
    // a run-time index, which puts the array into scratch memory (a store and a load of every
    // dword per chunk).  Not inline assembly either: the compiler inserts no wait states between
    // an MFMA and an assembly statement that overwrites one of the MFMA's result registers.
    const uint32_t m32 = (uint32_t)__builtin_amdgcn_sbfe((int)skew, 5, 1);
    const uint32_t m64 = (uint32_t)__builtin_amdgcn_sbfe((int)skew, 6, 1);
    uint32_t t2[C::NL];
#pragma unroll
    for (int i = 0; i < C::NL; ++i) t2[i] = mask_select(m32, t1[i], i + 1 < C::NL ? t1[i + 1] : 0u);
#pragma unroll
    for (int i = 0; i < C::ND; ++i) cw[i] = mask_select(m64, t2[i], i + 2 < C::NL ? t2[i + 2] : 0u);
  }
}

// Code stream of 32-column block jb of a chunk (3-bit codes widened to nibbles).
template <class C, int BITS>
__device__ inline void block_stream(const uint32_t (&cw)[C::ND], int jb, uint32_t (&st)[C::NW]) {
  if (BITS == 3) {
#pragma unroll
    for (int k = 0; k < C::NW; ++k) st[k] = expand3to4(get32<C::ND>(cw, jb * C::CB + 24 * k));
  } else {
#pragma unroll
    for (int k = 0; k < C::NW; ++k) st[k] = get32<C::ND>(cw, jb * C::CB + 32 * k);
  }
}

}  // namespace cbk
