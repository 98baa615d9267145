// Prefill GEMM:  Y[M, K] = X[M, N] . W_hat[K, N]^T on the gfx950 matrix cores.
//
// Workgroup tile 256 tokens x 256 weight rows, 64 input columns per stage, four wavefronts
// each owning a 128 x 128 sub-tile (4 x 4 blocks of v_mfma_f32_32x32x16_f16, 256 accumulator
// registers), one wavefront per SIMD.  Both operands are double-buffered in LDS (64 KB of
// activations, 72 KB of weights): while the matrix cores work on stage s, the same wavefronts
// dequantise the weights of stage s + 1 into the other buffer, and the activation tile is
// copied there from global memory without passing through registers.
//
// Operands.  The activation side is X' = fp16(x * col_scale / s_m), written once per call into
// the caller's workspace by a small row-wise kernel (bf16 inputs are widened exactly; the
// product is rounded once to fp16).  s_m is 1 unless token m holds a product of magnitude 2^15
// or more; then it is the power of two that brings the token's largest below 2^15, and the
// epilogue multiplies the token's outputs by it, so nothing saturates at fp16's 65504 and the
// scaling itself is exact.  The weight side is
// fp16((q - zero) * scale) for a kept column and exactly 0 for a pruned one, so
// Y = sum_j X'[m,j] * W'[k,j] carries two roundings of relative size 2^-12.  Feeding bf16
// operands instead would round to 2^-9, which alone exceeds the 1e-3 relative-Frobenius
// budget of this layer; the f16 and bf16 MFMA rates are identical.
//
// Weight decode.  Each of the 256 threads owns one weight row of the tile and decodes its
// 64 columns of the stage.  For 2/3/4-bit codes (bitmap layouts with 10, 16 or 23 of 32 kept,
// and the dense layouts) and for BLK1632_6, zero points <= 128, this is the byte-permute decoder
// of the decode kernel (selector table in LDS) followed by two packed-half operations per column
// pair; the remaining layouts (8-bit codes, larger zero points) go through the generic
// 32-column reader.
//
// Workgroups are ordered so that those running at the same time on one XCD (blockIdx % 8)
// share their token tile, which then stays in that XCD's L2.
//
// Reference semantics: cbk::gemm_tile (src/cobaltkernel/csrc/cobalt_gemm.cuh:243-609).
#pragma once
#include <atomic>
#include <type_traits>
#include "cbk_decode.h"

namespace cbk {

constexpr int GB_T = 256;       // tokens per workgroup tile (TI = 4); the TI = 1 kernels take 64
constexpr int GB_R = 256;       // weight rows per workgroup tile
constexpr int GB_K = 64;        // input columns per stage
constexpr int GB_P = GB_K + 8;  // LDS row pitch of the weight tile in halfs (144 B): conflict-free 16-byte reads
constexpr int GB_LUT = 256 * 8 * 8;   // selector table, 8 lane-private copies of 256 x 8 B
// one activation stage in LDS: 64 TI rows x 128 B, unpadded, swizzled
constexpr int gb_xbuf(int ti) { return 64 * ti * GB_K * 2; }
constexpr size_t gb_lds(int ti) { return (size_t)2 * gb_xbuf(ti) + (size_t)2 * GB_R * GB_P * 2 + GB_LUT; }

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

struct GbArgs {
  DMat m;
  const uint16_t* xp;      // X' fp16 [Mpad, Npad]
  const float* row_scale;  // [Mpad] per X': power of two each of its rows was divided by
  int rss;                 // elements between the row scales of two X'
  int M, Npad;
  void* y;
  int ydt;
  int64_t ldy;
  const void* bias;
  int tiles_t, tiles_r;
  int halves;              // gate/up matrix (par): 1 = write the gate outputs to columns [0, K/2) and the up outputs to
                           // [K/2, K) of y instead of interleaving them (whole 16-byte stores; for cbk_linear_act)
  int ti;                  // 32-token blocks per wavefront: 4 (256-token tiles) or 1 (64-token tiles)
  // par = 1: gate/up matrix, two col_scale vectors by row parity.  A workgroup then takes 256
  // rows of one parity out of 512 (rows r0 + 2 i + p), and X' of that parity's vector, which
  // starts xps elements after the other one.
  int par;
  size_t xps;
  // q|k|v matrix whose ranges start on row tiles: rows from vs0 on use the second X', rows from
  // vs1 on the third (both INT_MAX for any other matrix)
  int vs0, vs1;
  // split of the column range (PAR 3): nsplit workgroups per output tile take nst_part stages
  // each and leave float32 partial tiles [nsplit][.][part_ld] at part; a second kernel adds them
  int nsplit, nst_part;
  float* part;
  size_t part_stride;      // elements between the partial matrices
  int64_t part_ld;
};

// One wavefront-wide copy of 64 x 16 bytes from global memory straight into LDS (no VGPRs, no
// ds_write): lane l reads base + voff and its 16 bytes land at LDS byte lds + 16 * l.  The
// compiler does not know that this instruction counts on vmcnt or that it writes LDS; the
// kernel waits for it by hand before the barrier that publishes the stage.
__device__ inline void dma_x16(const void* base, uint32_t voff, uint32_t lds) {
  // base and lds are the same in every lane; say so, or they may arrive in vector registers
  const uint64_t b64 = (uint64_t)base;
  const uint64_t sbase = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b64) |
                         ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b64 >> 32)) << 32);
  lds = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
}

// eight signed bytes (q - z for a kept column, 0 for a pruned one) -> eight halfs times scale
__device__ inline uint4 bytes_to_halfs(uint32_t b0, uint32_t b1, h2_t s2) {
  // byte b (two's complement) -> u = b ^ 0x80 = b + 128 -> half bits 0x6400 | u = 1024 + 128 + b
  const uint32_t u0 = b0 ^ 0x80808080u, u1 = b1 ^ 0x80808080u;
  const uint32_t k = 0x64646464u;
  uint32_t w[4] = {__builtin_amdgcn_perm(k, u0, 0x04010400u), __builtin_amdgcn_perm(k, u0, 0x04030402u),
                   __builtin_amdgcn_perm(k, u1, 0x04010400u), __builtin_amdgcn_perm(k, u1, 0x04030402u)};
  const h2_t off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h2_t v = __builtin_bit_cast(h2_t, w[i]);
    v = (v + off) * s2;
    w[i] = __builtin_bit_cast(uint32_t, v);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// One wavefront's 128 x 128 accumulators -> y, 32 tokens at a time through LDS.  D[i][j] holds, in
// lane l and register r, token 8*(r/4) + 4*(l/32) + r%4 and weight row l%32 of its 32 x 32 block;
// turning the tile around in LDS makes the global stores whole 16-byte pieces of consecutive
// output columns: 256 B (f16) or 512 B (f32) per token.  Compile-time indexed and branch-free
// per element: the 256 accumulators make this straight-line code, and it has to stay small.
template <int YDT, int kstep, int TI>                            // local row i is output column row0 + kstep * i
__device__ inline void gb_epilogue(const GbArgs& a, v16f (&acc)[TI][4], uint8_t* smem, int lane, int wave, int tok0,
                                   int row0, const float* rs) {   // rs: the row scales of this tile's X'
  constexpr int ESZ = YDT == CBK_F32 ? 4 : 2;
  constexpr int PITCH = 128 * ESZ + 16;                          // bytes per token row in LDS
  constexpr int EPP = 16 / ESZ, PPR = 128 / EPP;                 // elements per 16-byte piece, pieces per row
  const int K = a.m.K;
  uint8_t* ep = smem + (size_t)wave * (32 * (128 * 4 + 16));
  uint8_t* epl = ep + 4 * (lane >> 5) * PITCH + (lane & 31) * ESZ;
  float bv[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int k = row0 + kstep * (32 * j + (lane & 31));
    bv[j] = 0.f;
    if (a.bias && k < K) bv[j] = load_act<YDT>(a.bias, k);
  }
  const bool vec_ok = ((a.ldy * ESZ) & 15) == 0 && (((uintptr_t)a.y) & 15) == 0;
#pragma unroll
  for (int i = 0; i < TI; ++i) {
    float ts[16];                                                  // token of register r: see above
#pragma unroll
    for (int r = 0; r < 16; ++r) ts[r] = rs[tok0 + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float v = acc[i][j][r] * ts[r] + bv[j];
        uint8_t* d = epl + (8 * (r >> 2) + (r & 3)) * PITCH + 32 * j * ESZ;
        if (YDT == CBK_F32) *(float*)d = v;
        else if (YDT == CBK_F16) *(uint16_t*)d = f2h(v);
        else *(__bf16*)d = (__bf16)v;                              // v_cvt_pk_bf16_f32: round to nearest even
      }
#pragma unroll
    for (int t = 0; t < 32 * PPR / 64; ++t) {
      const int pc = t * 64 + lane;
      const int row = pc / PPR, c = pc % PPR;
      const int tok = tok0 + 32 * i + row, k = row0 + kstep * (c * EPP);
      if (tok >= a.M || k >= K) continue;
      const uint8_t* src = ep + row * PITCH + c * 16;
      uint8_t* dst = (uint8_t*)a.y + ((size_t)tok * a.ldy + k) * ESZ;
      if (vec_ok && kstep == 1 && k + EPP <= K) *(uint4*)dst = *(const uint4*)src;
      else
        for (int e = 0; e < EPP && k + kstep * e < K; ++e) {
          if (ESZ == 4) ((float*)dst)[kstep * e] = ((const float*)src)[e];
          else ((uint16_t*)dst)[kstep * e] = ((const uint16_t*)src)[e];
        }
    }
  }
}

// BITS 2 / 3 / 4: byte-permute decoder for (BITS, KEEP, GRP), KEEP = 0 for the dense layouts.
// BITS 0: generic 32-column reader, any fixed-stride layout.
// PAR 0: one col_scale vector.  1: gate/up matrix (GbArgs::par).  2: q|k|v matrix (GbArgs::vs0, vs1).
// 3: one col_scale vector, column range split over several workgroups (GbArgs::nsplit).
// Three instantiations rather than run-time switches: the schedule of the main loop is tuned
// to the instruction and measurably shifts with every value that is added to it.
// TI: 32-token blocks per wavefront.  4: the 256-token tile described above.  2: a 128-token tile
// (each wavefront 64 tokens x 128 rows) for calls of 65 to 128 activation rows.  1: a 64-token tile
// (each wavefront 32 tokens x 128 rows) for calls of at most 64 activation rows, whose time is
// the weight decode: a quarter of the matrix instructions per stage, the same decode.
template <int BITS, int KEEP, int GRP, int PAR, int TI = 4>
__global__ __launch_bounds__(256) void gemm_big_kernel(GbArgs a) {
  constexpr int GB_XBUF = gb_xbuf(TI);
  constexpr bool FASTD = BITS != 0;
  using C = CodeCfg<FASTD ? BITS : 4, KEEP, FASTD ? GRP : 128>;
  constexpr bool BITMAP = FASTD && !C::DENSE;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // Xs [2][GB_T][64 halfs]: row r, logical 16-byte piece c at physical piece c ^ ((r >> 1) & 7)
  // (conflict-free 16-byte fragment reads without padding, which the direct copies cannot make)
  _Float16* Xs = (_Float16*)smem;
  _Float16* Ws = (_Float16*)(smem + 2 * GB_XBUF);                 // [2][GB_R][GB_P]
  uint2* lut = (uint2*)(Ws + 2 * GB_R * GB_P);                    // [256][8]
  const DMat& m = a.m;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wt = wave >> 1, wr = wave & 1;
  // XCD-aware order: blockIdx % 8 picks the XCD; give each XCD whole token tiles
  constexpr bool SPLIT = PAR == 3;
  const int nb = a.tiles_t * a.tiles_r * (SPLIT ? a.nsplit : 1);
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int per = (nb + 7) >> 3;
  const int lin = xcd * per + idx;                                 // token-tile-major linear id
  if (lin >= nb) return;
  const int part = SPLIT ? lin % a.nsplit : 0, tile = SPLIT ? lin / a.nsplit : lin;
  const int tt = tile / a.tiles_r, tr = tile % a.tiles_r;
  constexpr int kstep = PAR == 1 ? 2 : 1;                         // row stride of this workgroup's rows
  const int pp = PAR == 1 ? (tr & 1) : 0;                         // and their parity
  const int t0 = tt * (64 * TI), r0 = PAR == 1 ? (tr >> 1) * (2 * GB_R) + pp : tr * GB_R;
  const int N = m.N, Npad = a.Npad;
  // stages of this workgroup: all of them, or its part of them; a multiple of 4 either way;
  // stages past N see X' = 0
  const int s_begin = SPLIT ? part * a.nst_part : 0;
  const int nst = SPLIT ? (Npad / GB_K - s_begin < a.nst_part ? Npad / GB_K - s_begin : a.nst_part) : Npad / GB_K;
  const int c_begin = s_begin >> 1;                               // first 128-column chunk
  const int nch = N >> 7;                                         // 128-column chunks of the weight rows

  if (BITMAP) {
    const uint2 e = make_selectors((uint32_t)tid, C::SEL_KIND);
#pragma unroll
    for (int j = 0; j < 8; ++j) lut[tid * 8 + j] = e;
  }
  const uint32_t l8 = lane & 7;

  v16f acc[TI][4];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // this thread's weight row
  const int wrow = r0 + kstep * tid;
  const bool wok = wrow < m.K;
  const int wrc = wok ? wrow : m.K - 1;
  const RowView rv = row_view(m, wrc);
  const size_t meta0 = meta_index(m, wrc, 0), meta_step = m.tiled ? 16 : 1;
  // Activation tile: wavefront w copies rows 16 TI w .. 16 TI (w+1) - 1 of every stage with 2 TI
  // direct copies of eight rows each; lane l of copy q takes row 16 TI w + 8q + l/8 and fills
  // physical piece l%8 of it, i.e. fetches logical piece (l%8) ^ ((4q + l/16) & 7).  That is one
  // of two values per lane (q even / odd), so two lane offsets and a scalar base per copy suffice.
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t xvo_e = (uint32_t)((lane >> 3) * Npad * 2 + (((lane & 7) ^ (lane >> 4)) * 16));
  const uint32_t xvo_o = (uint32_t)((lane >> 3) * Npad * 2 + (((lane & 7) ^ (4 + (lane >> 4))) * 16));
  const int xv = PAR == 1 ? pp : PAR == 2 ? (r0 >= a.vs0 ? 1 : 0) + (r0 >= a.vs1 ? 1 : 0) : 0;   // which col_scale vector
  const uint8_t* xsb = (const uint8_t*)(a.xp + (size_t)xv * a.xps + (size_t)(t0 + 16 * TI * wv) * Npad + (size_t)s_begin * GB_K);
  const uint32_t xlds0 = (uint32_t)(uintptr_t)Xs + (uint32_t)wv * (2048u * TI);
  auto dma_x = [&](int s, int buf) {                              // stage s -> Xs[buf]
    const uint8_t* sb = xsb + (size_t)s * (GB_K * 2);
    const uint32_t ld = xlds0 + (uint32_t)buf * GB_XBUF;
#pragma unroll
    for (int q = 0; q < 2 * TI; ++q)
      dma_x16(sb + (size_t)q * 8 * Npad * 2, (q & 1) ? xvo_o : xvo_e, ld + q * 1024);
  };
  // fragment reads: this lane's row inside a 32-row block and its four swizzled piece offsets
  const uint32_t xsw = ((lane & 31) >> 1) & 7;
  uint32_t xpc[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) xpc[kk] = (((2 * kk + (lane >> 5)) ^ xsw) * 16);

  // one 128-column chunk of this thread's weight row: two stages' worth
  struct WChunk {
    uint32_t m[4];                       // bitmap
    uint32_t raw[C::NL];                 // code dwords as loaded (whole 16-byte units)
    uint32_t c[C::ND];                   // code bits, first bit of the chunk at bit 0
    uint32_t z;                          // zero points of the chunk's groups, one per byte
    float s[C::NGC];
    uint32_t ci;                         // chunk index the units were loaded for
    uint32_t h2[C::HI2 ? 4 : 1];         // BLK1632_6: high bit pairs, one dword per block
  };
  WChunk wA, wB;
  uint32_t st[C::NW];                                             // code stream of the block being decoded

  auto load_chunk = [&](int c, WChunk& w) {
    if (!FASTD) return;
    c += c_begin;
    c = c < nch ? c : nch - 1;
    w.ci = (uint32_t)c;
    if (BITMAP) {
      const uint4 mk = *(const uint4*)rv.unit((uint32_t)c);                         // 16 B of bitmap
      w.m[0] = mk.x; w.m[1] = mk.y; w.m[2] = mk.z; w.m[3] = mk.w;
    }
    const uint32_t u0 = (m.code_off >> 4) + (C::VEC16 ? (uint32_t)c * (C::CHB / 128) : (((uint32_t)c * C::CHB) >> 7));
#pragma unroll
    for (int i = 0; i < C::NL / 4; ++i) {
      const uint4 v = *(const uint4*)rv.unit(u0 + i);
      w.raw[4 * i] = v.x; w.raw[4 * i + 1] = v.y; w.raw[4 * i + 2] = v.z; w.raw[4 * i + 3] = v.w;
    }
    if (C::HI2) {                                                   // the plane behind mask and nibbles
      const uint4 v = *(const uint4*)rv.unit(3u * (uint32_t)nch + (uint32_t)c);
      w.h2[0] = v.x; w.h2[1] = v.y; w.h2[2] = v.z; w.h2[3] = v.w;
    }
    const size_t mi = meta0 + (size_t)c * C::NGC * meta_step;
    w.z = m.zero[mi];
    w.s[0] = h2f(m.scale[mi]);
    if (C::NGC == 2) {
      w.z |= (uint32_t)m.zero[mi + meta_step] << 8;
      w.s[1] = h2f(m.scale[mi + meta_step]);
    }
  };

  // selectors of mask byte b8 (0..7) of half h of a chunk (bitmap layouts only)
  auto fetch_sel = [&](const WChunk& w, int h, int b8) -> uint2 {
    if (!BITMAP) return make_uint2(0, 0);
    const int jb = 8 * h + b8;                                     // mask byte of the chunk, 0..15
    const uint32_t mb = (w.m[jb >> 2] >> (8 * (jb & 3))) & 0xFFu;
    return lut[mb * 8 + l8];
  };
  // decode mask byte b8 (8 columns) of stage s = half h of chunk w into Ws[buf]
  auto store_w_byte = [&](int s, WChunk& w, int h, int buf, int b8, uint2 sel) {
    _Float16* dst = Ws + (size_t)buf * GB_R * GB_P + tid * GB_P + b8 * 8;
    if (!FASTD) {
      if (b8 & 3) return;                                         // the generic reader works on 32 columns
      uint32_t packed[16];
      if (wok) {
        int q[32];
        int t = ((s + s_begin) * GB_K >> 5) + (b8 >> 2);
        t = t < (N >> 5) ? t : (N >> 5) - 1;
        const uint32_t keep = decode_block32(m, rv, t, q);
        const int g = (t * BLOCK) / m.group;
        const float sc = h2f(m.scale[meta_index(m, wrc, g)]);
        const float z = (float)m.zero[meta_index(m, wrc, g)];
        const bool dense = family_of(m.layout) == FAM_DENSE;
#pragma unroll
        for (int p = 0; p < 32; p += 2) {
          float v0 = __fmul_rn((float)q[p] - z, sc), v1 = __fmul_rn((float)q[p + 1] - z, sc);
          if (!dense) { v0 = ((keep >> p) & 1u) ? v0 : 0.f; v1 = ((keep >> (p + 1)) & 1u) ? v1 : 0.f; }
          packed[p >> 1] = (uint32_t)f2h(v0) | ((uint32_t)f2h(v1) << 16);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) packed[e] = 0;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
        ((uint4*)dst)[e] = make_uint4(packed[4 * e], packed[4 * e + 1], packed[4 * e + 2], packed[4 * e + 3]);
      return;
    }
    if (h == 0 && b8 == 0) align_chunk_codes<C>(w.raw, w.ci, w.c);  // once per chunk, at its first use
    const int blk = 2 * h + (b8 >> 2);                              // 32-column block of the chunk
    const int jj = b8 & 3;                                          // mask byte inside the block
    if (jj == 0) block_stream<C, BITS>(w.c, blk, st);               // once per block
    const int gi = C::NGC == 2 ? h : 0;                             // quantisation group of this stage
    const _Float16 sh = (_Float16)(wok ? w.s[gi] : 0.f);
    const h2_t s2 = {sh, sh};
    const uint32_t nz = 0x80808080u - ((w.z >> (8 * gi)) & 0xFFu) * 0x01010101u;
    uint32_t p0, p1, b0, b1;
    if (BITMAP) {
      const uint32_t mw = w.m[blk];
      const uint32_t r = jj == 0 ? 0u : (uint32_t)__builtin_popcount(mw & ((1u << (8 * jj)) - 1u));
      const uint32_t cwin = jj == 0 ? st[0] : window<C::NW>(st, r * C::SB);
      if (C::HI2) {
        uint32_t h0, h1;
        hi2_pools(w.h2[C::HI2 ? blk : 0], r, h0, h1);
        p0 = bias_pool((cwin & 0x0F0F0F0Fu) | h0, nz);
        p1 = bias_pool(((cwin >> 4) & 0x0F0F0F0Fu) | h1, nz);
      } else if (C::SB == 4) {
        p0 = bias_pool(cwin & 0x0F0F0F0Fu, nz);
        p1 = bias_pool((cwin >> 4) & 0x0F0F0F0Fu, nz);
      } else {
        const uint32_t lo16 = cwin & 0xFFFFu;
        const uint32_t t2 = (lo16 << 14) | lo16;
        p0 = bias_pool(t2 & 0x03030303u, nz);
        p1 = bias_pool((t2 >> 4) & 0x03030303u, nz);
      }
      b0 = perm(p1, p0, sel.x);
      b1 = perm(p1, p0, sel.y);
    } else if (C::SB == 4) {                                       // dense 4-bit, or 3-bit widened to nibbles
      const uint32_t cwin = st[jj];
      p0 = bias_pool(cwin & 0x0F0F0F0Fu, nz);                      // even columns
      p1 = bias_pool((cwin >> 4) & 0x0F0F0F0Fu, nz);               // odd columns
      b0 = perm(p1, p0, 0x05010400u);
      b1 = perm(p1, p0, 0x07030602u);
    } else {                                                       // dense 2-bit: 16 codes per dword
      const uint32_t lo16 = (st[jj >> 1] >> (16 * (jj & 1))) & 0xFFFFu;
      const uint32_t t2 = (lo16 << 14) | lo16;
      p0 = bias_pool(t2 & 0x03030303u, nz);                        // c0 c4 c1 c5
      p1 = bias_pool((t2 >> 4) & 0x03030303u, nz);                 // c2 c6 c3 c7
      b0 = perm(p1, p0, 0x06040200u);
      b1 = perm(p1, p0, 0x07050301u);
    }
    *(uint4*)dst = bytes_to_halfs(b0, b1, s2);
  };

  // fragment registers, two sets; set 0 of the next stage is loaded at the end of the current one
  v8h af[2][TI], bf[2][4];
  auto read_frags = [&](int buf, int kk, int set) {
    const uint8_t* xb = (const uint8_t*)Xs + (size_t)buf * GB_XBUF + (32 * TI * wt + (lane & 31)) * 128;
    const _Float16* wb = Ws + (size_t)buf * GB_R * GB_P + (128 * wr + (lane & 31)) * GB_P + 8 * (lane >> 5);
#pragma unroll
    for (int i = 0; i < TI; ++i) af[set][i] = *(const v8h*)(xb + 4096 * i + xpc[kk]);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[set][j] = *(const v8h*)(wb + 32 * j * GB_P + 16 * kk);
  };

  // ---- prologue: chunk 0 into registers and stage 0 into buffer 0; then, in the order every
  // stage leaves them, the copies of stage 1 and the loads of chunk 1
  dma_x(0, 0);
  load_chunk(0, wA);
  __syncthreads();                                                // selector table visible
#pragma unroll
  for (int b8 = 0; b8 < 8; ++b8) store_w_byte(0, wA, 0, 0, b8, fetch_sel(wA, 0, b8));
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  read_frags(0, 0, 0);
  dma_x(nst > 1 ? 1 : 0, 1);
  load_chunk(1, wB);
  uint2 selc[3];                                                  // selectors of the mask bytes decoded next
#pragma unroll
  for (int i = 0; i < 3; ++i) selc[i] = fetch_sel(wA, 1, i);

  // One stage = four phases of 16 MFMAs on buffer s % 2.  Phases 0-2 also decode the weights of
  // stage s + 1 (half HD of chunk wd; mask bytes 0-2, 3-5, 6-7) into the other buffer between
  // their MFMAs, fetching the selectors of the following phase (at the end: of bytes 0-2 of half
  // HN of chunk wn) a phase early.  Phase 3 first waits for the direct copies of stage s + 1
  // (issued a stage ago) and passes the barrier, then starts the fragment reads of stage s + 1,
  // the direct copies of stage s + 2 and, with LOADW, the loads of weight chunk `cl`, and only
  // then issues its 16 MFMAs from registers: the LDS latency of the next stage hides under them.
  // No branches inside.
  constexpr int NB0 = 3, NB1 = 3;                                 // mask bytes decoded in phases 0 and 1
  auto stage = [&](int s, auto loadw_tag, WChunk& wd, auto hd_tag, const WChunk& wn, auto hn_tag, WChunk& wl, int cl) {
    constexpr bool LOADW = decltype(loadw_tag)::value;
    constexpr int HD = decltype(hd_tag)::value, HN = decltype(hn_tag)::value;
    const int buf = s & 1;
#pragma unroll
    for (int kk = 0; kk < GB_K / 16; ++kk) {
      const int c = kk & 1, n = c ^ 1;
      if (kk < 3) {
        read_frags(buf, kk + 1, n);
        uint2 seln[3];
        if (kk == 0) {
#pragma unroll
          for (int i = 0; i < NB1; ++i) seln[i] = fetch_sel(wd, HD, NB0 + i);
#pragma unroll
          for (int i = 0; i < NB0; ++i) store_w_byte(s + 1, wd, HD, buf ^ 1, i, selc[i]);
        } else if (kk == 1) {
#pragma unroll
          for (int i = 0; i < 8 - NB0 - NB1; ++i) seln[i] = fetch_sel(wd, HD, NB0 + NB1 + i);
#pragma unroll
          for (int i = 0; i < NB1; ++i) store_w_byte(s + 1, wd, HD, buf ^ 1, NB0 + i, selc[i]);
        } else {
#pragma unroll
          for (int i = 0; i < NB0; ++i) seln[i] = fetch_sel(wn, HN, i);
#pragma unroll
          for (int i = 0; i < 8 - NB0 - NB1; ++i) store_w_byte(s + 1, wd, HD, buf ^ 1, NB0 + NB1 + i, selc[i]);
        }
#pragma unroll
        for (int i = 0; i < 3; ++i) selc[i] = seln[i];
      } else {
        // the direct copies of stage s + 1 must have landed before the barrier publishes them
        // (the weight chunk loads of the previous stage wait here as well: they were issued a
        // whole stage ago, and counting them out of the wait would rest on how many load
        // instructions the compiler keeps)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        read_frags(buf ^ 1, 0, 0);
        dma_x(s + 2 < nst ? s + 2 : nst - 1, buf);
        if (LOADW) load_chunk(cl, wl);
      }
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[c][i], bf[c][j], acc[i][j], 0, 0, 0);
      if (kk < 3) {
#pragma unroll
        for (int g = 0; g < 4 * TI; ++g) {                        // one MFMA, then a slice of the decode
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (kk == 2) __builtin_amdgcn_sched_group_barrier(0x002, 16 / TI, 0);
          else __builtin_amdgcn_sched_group_barrier(0x002, 20 / TI, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Four stages per trip (two chunks): stage 2p decodes the upper half of chunk p and, in its
  // last phase, loads chunk p+2 into the registers chunk p has just left; stage 2p+1 decodes the
  // lower half of chunk p+1.  The loads so have a stage and three phases until their first use
  // (the selectors of chunk p+2 at the end of stage 2p+2); issued a stage later, where the
  // kernel first had them, their latency from HBM showed: 3-4 % of the run time.
  using T = std::true_type; using Fl = std::false_type;
  using H0 = std::integral_constant<int, 0>; using H1 = std::integral_constant<int, 1>;
  for (int s = 0; s < nst; s += 4) {
    const int p = s >> 1;
    stage(s,     T{},  wA, H1{}, wB, H0{}, wA, p + 2);
    stage(s + 1, Fl{}, wB, H0{}, wB, H1{}, wA, 0);
    stage(s + 2, T{},  wB, H1{}, wA, H0{}, wB, p + 3);
    stage(s + 3, Fl{}, wA, H0{}, wA, H1{}, wB, 0);
  }
  // the last stage issued copies of a stage that does not exist: let them land before the
  // epilogue reuses LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  const int tok0 = t0 + 32 * TI * wt, row0 = r0 + kstep * 128 * wr;
  const float* rs = a.row_scale + (size_t)xv * a.rss;
  if (SPLIT) {                                                    // float32 partial tile, no bias
    GbArgs b = a;
    b.y = a.part + (size_t)part * a.part_stride;
    b.ldy = a.part_ld;
    b.bias = nullptr;
    gb_epilogue<CBK_F32, 1, TI>(b, acc, smem, lane, wave, tok0, row0, rs);
    return;
  }
  if (PAR == 1 && a.halves) {
    // this workgroup's rows are one parity of the matrix: consecutive columns of that half of y
    GbArgs b = a;
    const int K2 = a.m.K >> 1;
    b.y = (uint8_t*)a.y + (size_t)pp * K2 * (a.ydt == CBK_F32 ? 4 : 2);
    b.m.K = K2;
    b.bias = nullptr;
    const int hrow0 = (r0 >> 1) + 128 * wr;
    if (a.ydt == CBK_F32) gb_epilogue<CBK_F32, 1, TI>(b, acc, smem, lane, wave, tok0, hrow0, rs);
    else if (a.ydt == CBK_F16) gb_epilogue<CBK_F16, 1, TI>(b, acc, smem, lane, wave, tok0, hrow0, rs);
    else gb_epilogue<CBK_BF16T, 1, TI>(b, acc, smem, lane, wave, tok0, hrow0, rs);
    return;
  }
  if (a.ydt == CBK_F32) gb_epilogue<CBK_F32, kstep, TI>(a, acc, smem, lane, wave, tok0, row0, rs);
  else if (a.ydt == CBK_F16) gb_epilogue<CBK_F16, kstep, TI>(a, acc, smem, lane, wave, tok0, row0, rs);
  else gb_epilogue<CBK_BF16T, kstep, TI>(a, acc, smem, lane, wave, tok0, row0, rs);
}

template <int BITS, int KEEP, int GRP, int PAR, int TI>
static int launch_big_par(const GbArgs& a, int blocks, hipStream_t st) {
  auto kern = gemm_big_kernel<BITS, KEEP, GRP, PAR, TI>;
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), gb_lds(TI), st, a);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

template <int BITS, int KEEP, int GRP, int TI>
static int launch_big_ti(const GbArgs& a, int blocks, hipStream_t st) {
  if (a.par) return launch_big_par<BITS, KEEP, GRP, 1, TI>(a, blocks, st);
  if (a.vs0 != 0x7fffffff) return launch_big_par<BITS, KEEP, GRP, 2, TI>(a, blocks, st);
  if (a.nsplit > 1) return launch_big_par<BITS, KEEP, GRP, 3, TI>(a, blocks, st);
  return launch_big_par<BITS, KEEP, GRP, 0, TI>(a, blocks, st);
}

template <int BITS, int KEEP, int GRP>
static int launch_big_cfg(const GbArgs& a, int blocks, hipStream_t st) {
  return a.ti == 1 ? launch_big_ti<BITS, KEEP, GRP, 1>(a, blocks, st)
       : a.ti == 2 ? launch_big_ti<BITS, KEEP, GRP, 2>(a, blocks, st) : launch_big_ti<BITS, KEEP, GRP, 4>(a, blocks, st);
}

// the (keep, group) instantiations of one code width and one token tile (a translation unit each:
// the 32 kernels of such a set are what one compiler process takes a minute and a half for)
template <int BITS, int TI>
static int launch_big_bits(const GbArgs& a, int keep, int group, int blocks, hipStream_t st) {
#define CBK_GB_CASE(KEEP)                                                                            \
  case KEEP: return group == 64 ? launch_big_ti<BITS, KEEP, 64, TI>(a, blocks, st)                   \
                                : launch_big_ti<BITS, KEEP, 128, TI>(a, blocks, st);
  switch (keep) {
    CBK_GB_CASE(0) CBK_GB_CASE(10) CBK_GB_CASE(16) CBK_GB_CASE(23)
    default: return CBK_ERR_UNSUPPORTED;
  }
#undef CBK_GB_CASE
}

}  // namespace cbk
