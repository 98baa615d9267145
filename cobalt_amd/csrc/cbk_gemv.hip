// Decode GEMV / skinny GEMM (1 <= M <= 8) on the gfx950 int8 matrix cores.
//
// Idea.  At 8 TB/s and ~3 bits per weight the chip must consume ~20e12 weights per second,
// which leaves about two vector-ALU instructions per weight: a per-weight convert + FMA
// dequantiser cannot keep up.  So the weights stay integers.  Every lane decodes 128
// consecutive columns of ONE weight row into signed bytes (q - zero for a kept column, 0
// for a pruned one) sixteen at a time, and hands each 16-byte fragment to
// v_mfma_i32_16x16x64_i8 as the B operand.  The A operand is the activation vector in
// block fixed point: per 128-column chunk, x' = x * col_scale is written as
// delta * (256*hi + lo) with two int8 digits (|x' - delta*X| <= max|x'| / 65024).  The
// matrix core produces exact int32 dot products per (row, chunk, digit); one float FMA per
// row and quantisation group applies scale * delta.  A pruned column multiplies a literal
// zero byte, so it contributes exactly 0 whatever the zero point holds.
//
// Work decomposition.  A wavefront owns a tile of 16 weight rows; lane l works on row l%16
// and on the 128-column chunk 4*S + l/16 of macro-step S (512 columns).  The four lane
// quarters are four different quantisation groups, which one MFMA would add up; the rows of
// the A operand therefore carry (activation row, quarter, digit) variants that are non-zero
// in one quarter only, and the 16x16 result keeps the groups apart.  The eight wavefronts of
// a workgroup split the macro-steps of a tile and combine through LDS in a fixed order, so
// results are run-to-run identical.  Workgroups are persistent over row tiles; the
// activation digits and the byte-permute selector table live in LDS for the whole launch.
//
// Expansion of the bitmap.  For one mask byte (8 columns, r survivors before it in its
// 32-column block) the survivor codes r .. r+7 are shifted out of the block's code bits,
// spread to one code per byte (two dwords = the 8-byte pool of v_perm_b32), biased to
// q - zero, and v_perm_b32 with a selector from a 256-entry table (indexed by the mask
// byte) drops each survivor into its column and a constant 0 into every pruned column.
//
// Reference semantics: cbk::gemv_blk1632_multi / gemv_dense4_multi
// (src/cobaltkernel/csrc/cobalt_gemv.cuh:617-712, :839-1123): same sums, other machinery.
#include <atomic>
#include "cbk_device.h"

namespace cbk {

constexpr int GV_WAVES = 8;
constexpr int GV_THREADS = GV_WAVES * 64;
constexpr int LUT_LANES = 16;                 // lane-private copies of the selector table
constexpr int LUT_BYTES = 256 * LUT_LANES * 8;
constexpr int ZERO_BYTES = 256;
constexpr int X_LDS_BUDGET = 112 * 1024;      // activation digits: M * 2 * N bytes
constexpr int GV_MAX_M = 8;

// ------------------------------------------------------------------ selector tables
struct SelTable { uint32_t lo[256], hi[256]; };

// kind 0: pool = {even-rank codes (bytes 0-3), odd-rank codes (bytes 4-7)}   (4-bit codes)
// kind 1: pool = {c0,c4,c1,c5 | c2,c6,c3,c7}                                   (2-bit codes)
constexpr SelTable make_table(int kind) {
  SelTable t{};
  for (int mb = 0; mb < 256; ++mb) {
    uint32_t sel[8] = {};
    int r = 0;
    for (int p = 0; p < 8; ++p) {
      if ((mb >> p) & 1) {
        sel[p] = kind == 0 ? (uint32_t)((r >> 1) + 4 * (r & 1)) : (uint32_t)(((r & 3) << 1) | (r >> 2));
        ++r;
      } else {
        sel[p] = 0x0Cu;                        // v_perm_b32: constant 0x00
      }
    }
    t.lo[mb] = sel[0] | (sel[1] << 8) | (sel[2] << 16) | (sel[3] << 24);
    t.hi[mb] = sel[4] | (sel[5] << 8) | (sel[6] << 16) | (sel[7] << 24);
  }
  return t;
}
__device__ const SelTable g_sel4 = make_table(0);
__device__ const SelTable g_sel2 = make_table(1);

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

// pool bytes holding a code q each  ->  signed bytes q - z   (z <= 128, carried in nz)
__device__ inline uint32_t bias_pool(uint32_t codes, uint32_t nz) { return (codes + nz) ^ 0x80808080u; }

// ------------------------------------------------------------------ kernel configuration
// BITS: code width.  KEEP: survivors per 32 columns, 0 = dense family.  GRP: group size.
// MP: MFMA passes per fragment = ceil(M / 2).
template <int BITS, int KEEP, int GRP, int MP>
struct Cfg {
  static constexpr bool DENSE = KEEP == 0;
  static constexpr int CB = DENSE ? 32 * BITS : KEEP * BITS;      // code bits per 32-column block
  static constexpr int CHB = 4 * CB;                              // per 128-column chunk
  static constexpr bool ALIGNED = CHB % 32 == 0;
  static constexpr int ND = (CHB + 31) / 32;                      // dwords of chunk code bits
  static constexpr int NL = ALIGNED ? ND : ND + 1;                // dwords loaded (skew)
  static constexpr bool VEC16 = CHB % 128 == 0;                   // 16-byte aligned chunks
  static constexpr int NIB = DENSE ? 32 : KEEP;                   // codes per block
  static constexpr int SB = BITS == 3 ? 4 : BITS;                 // stream code width after expansion
  static constexpr int NW = (NIB * SB + 31) / 32;                 // dwords of a block's code stream
  static constexpr int NGC = 128 / GRP;                           // groups per chunk (1 or 2)
};

struct GvArgs {
  DMat m;
  const uint16_t* x;
  int64_t ldx;
  int M;
  void* y;
  int ydt;
  int64_t ldy;
  const void* bias;
  int xdt;
  int ntiles;
};

// Column order of the activation digits inside a 16-column fragment (dense family only):
// the byte order in which the spread codes come out without a permute.
template <int BITS, bool DENSE>
__device__ constexpr int frag_col(int bi) {
  if (!DENSE) return bi;
  if (BITS == 2) return (bi >> 2) + 4 * (bi & 3);                                 // byte 4k+j <- column k+4j
  return ((bi >> 3) << 3) + 2 * (bi & 3) + ((bi >> 2) & 1);                       // even | odd per 8
}

// ------------------------------------------------------------------ the kernel
template <int BITS, int KEEP, int GRP, int MP>
__global__ __launch_bounds__(GV_THREADS) void gemv_mfma_kernel(GvArgs a) {
  using C = Cfg<BITS, KEEP, GRP, MP>;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const DMat& m = a.m;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int N = m.N, NCH = N >> 7;
  uint2* lut = (uint2*)smem;
  uint8_t* zreg = smem + LUT_BYTES;
  int8_t* xq = (int8_t*)(zreg + ZERO_BYTES);                       // [M][2][N]
  float* delta = (float*)(xq + (size_t)a.M * 2 * N);               // [M][NCH + 4]
  float* red = delta + (size_t)a.M * (NCH + 4);                    // [2][GV_WAVES][GV_MAX_M][16]

  // ---- selector table, one copy per lane%16 so that a wavefront's lookups do not collide
  {
    const SelTable& t = (BITS == 2 && !C::DENSE) ? g_sel2 : g_sel4;
    for (int i = tid; i < 256 * LUT_LANES; i += GV_THREADS) lut[i] = make_uint2(t.lo[i / LUT_LANES], t.hi[i / LUT_LANES]);
    if (tid < ZERO_BYTES / 4) ((uint32_t*)zreg)[tid] = 0u;
  }
  // ---- activations -> block fixed point.  One item = 16 columns; 8 items = one chunk.
  {
    const int items = a.M * (N >> 4);
    for (int it = tid; it < ((items + 7) & ~7); it += GV_THREADS) {
      const bool ok = it < items;
      const int mi = ok ? it / (N >> 4) : 0, c16 = ok ? it % (N >> 4) : 0;
      float xv[16];
      const uint16_t* xp = a.x + (size_t)mi * a.ldx + c16 * 16;
      const uint16_t* cp = m.cs ? m.cs + c16 * 16 : nullptr;
      uint4 xr[2] = {((const uint4*)xp)[0], ((const uint4*)xp)[1]};
      uint4 cr[2];
      if (cp) { cr[0] = ((const uint4*)cp)[0]; cr[1] = ((const uint4*)cp)[1]; }
      const uint32_t* xw = (const uint32_t*)xr;
      const uint32_t* cw = (const uint32_t*)cr;
      float mx = 0.f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint16_t xb = (uint16_t)(xw[e >> 1] >> (16 * (e & 1)));
        float v = a.xdt == CBK_F16 ? h2f(xb) : bf2f(xb);
        if (cp) v *= h2f((uint16_t)(cw[e >> 1] >> (16 * (e & 1))));
        xv[e] = ok ? v : 0.f;
        mx = fmaxf(mx, fabsf(xv[e]));
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      const float d = mx > 0.f ? mx / 32512.f : 1.f;
      const float inv = 1.f / d;
      uint32_t hw[4] = {0, 0, 0, 0}, lw[4] = {0, 0, 0, 0};
#pragma unroll
      for (int bi = 0; bi < 16; ++bi) {
        const int X = (int)rintf(xv[frag_col<BITS, C::DENSE>(bi)] * inv);
        const int h = (X + 128) >> 8;
        const int l = X - (h << 8);
        hw[bi >> 2] |= ((uint32_t)h & 0xFFu) << (8 * (bi & 3));
        lw[bi >> 2] |= ((uint32_t)l & 0xFFu) << (8 * (bi & 3));
      }
      if (ok) {
        *(uint4*)(xq + ((size_t)mi * 2 + 0) * N + c16 * 16) = make_uint4(hw[0], hw[1], hw[2], hw[3]);
        *(uint4*)(xq + ((size_t)mi * 2 + 1) * N + c16 * 16) = make_uint4(lw[0], lw[1], lw[2], lw[3]);
        if ((c16 & 7) == 0) delta[mi * (NCH + 4) + (c16 >> 3)] = d;
      }
    }
    if (tid < a.M * 4) delta[(tid >> 2) * (NCH + 4) + NCH + (tid & 3)] = 0.f;   // chunks past N
  }
  __syncthreads();

  const int wr = lane & 15, kq = lane >> 4;            // weight row in tile / lane quarter
  const int nS = (NCH + 3) >> 2;
  const uint32_t l16 = lane & (LUT_LANES - 1);
  // role of this lane's row in the A operand: variant i = lane%16
  const int a_mloc = wr >> 3, a_slice = (wr >> 1) & 3, a_dig = wr & 1;
  // role of this lane in the result: activation row 2p + kq/2, slices 2*(kq&1) and +1
  const int o_mloc = kq >> 1, o_s0 = 2 * (kq & 1);
  int buf = 0;

  for (int tile = blockIdx.x; tile < a.ntiles; tile += gridDim.x) {
    const int row = tile * 16 + wr;
    const int rowc = row < m.K ? row : m.K - 1;
    const uint8_t* rowp = m.data + (size_t)rowc * m.stride;
    const uint16_t* scp = m.scale + (size_t)rowc * m.G;
    const uint8_t* zp = m.zero + (size_t)rowc * m.G;
    float ysum[MP];
#pragma unroll
    for (int p = 0; p < MP; ++p) ysum[p] = 0.f;

    for (int S = wave; S < nS; S += GV_WAVES) {
      const int chunk = 4 * S + kq;
      const bool valid = chunk < NCH;
      const int chc = valid ? chunk : NCH - 1;
      // ---- loads: bitmap, code bits, zero points, scales
      uint32_t mk[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
      if (!C::DENSE) {
        const uint4 v = *(const uint4*)(rowp + 16 * chc);
        mk[0] = v.x; mk[1] = v.y; mk[2] = v.z; mk[3] = v.w;
      }
      uint32_t raw[C::NL];
      uint32_t skew = 0;
      {
        const uint8_t* plane = rowp + m.code_off;
        if (C::VEC16) {
          const uint4* p = (const uint4*)(plane + (size_t)chc * (C::CHB / 8));
#pragma unroll
          for (int i = 0; i < C::ND / 4; ++i) { const uint4 v = p[i]; raw[4 * i] = v.x; raw[4 * i + 1] = v.y; raw[4 * i + 2] = v.z; raw[4 * i + 3] = v.w; }
        } else {
          const uint32_t sb = (uint32_t)chc * C::CHB;
          const uint32_t* p = (const uint32_t*)plane + (sb >> 5);
          skew = sb & 31u;
#pragma unroll
          for (int i = 0; i < C::NL; ++i) raw[i] = p[i];
        }
      }
      uint32_t zraw;
      if (C::NGC == 1) zraw = zp[chc];
      else zraw = *(const uint16_t*)(zp + 2 * chc);
      // scales of the two chunks this lane post-processes
      float sc[2][C::NGC];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        int ch = 4 * S + o_s0 + s;
        ch = ch < NCH ? ch : NCH - 1;
#pragma unroll
        for (int g = 0; g < C::NGC; ++g) sc[s][g] = h2f(scp[ch * C::NGC + g]);
      }
      // ---- A operand addresses (activation digits of this lane's own columns, or zeros)
      uint32_t aaddr[MP];
#pragma unroll
      for (int p = 0; p < MP; ++p) {
        const int mi = 2 * p + a_mloc;
        const bool on = valid && a_slice == kq && mi < a.M;
        aaddr[p] = on ? (uint32_t)((xq - (int8_t*)smem) + ((size_t)mi * 2 + a_dig) * N + chunk * 128)
                      : (uint32_t)(zreg - smem);
      }
      // ---- align the chunk's code bits
      uint32_t cw[C::ND];
#pragma unroll
      for (int i = 0; i < C::ND; ++i)
        cw[i] = C::ALIGNED ? raw[i] : __builtin_amdgcn_alignbit(raw[i + 1], raw[i], skew);

      v4i acc[MP];
#pragma unroll
      for (int p = 0; p < MP; ++p) acc[p] = (v4i){0, 0, 0, 0};

#pragma unroll
      for (int jb = 0; jb < 4; ++jb) {
        // code stream of block jb, SB bits per code
        uint32_t st[C::NW];
        if (BITS == 3) {
#pragma unroll
          for (int k = 0; k < C::NW; ++k) st[k] = expand3to4(get32<C::ND>(cw, jb * C::CB + 24 * k));
        } else {
#pragma unroll
          for (int k = 0; k < C::NW; ++k) st[k] = get32<C::ND>(cw, jb * C::CB + 32 * k);
        }
        const uint32_t z = (C::NGC == 1) ? zraw : ((zraw >> (8 * (jb >> 1))) & 0xFFu);
        const uint32_t nz = 0x80808080u - z * 0x01010101u;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          uint32_t bfrag[4];
#pragma unroll
          for (int jj2 = 0; jj2 < 2; ++jj2) {
            const int jj = 2 * half + jj2;                       // mask byte inside the block
            uint32_t p0, p1;
            if (C::DENSE) {
              // 8 codes at a compile-time position
              if (C::SB == 4) {
                const uint32_t w = st[jj];
                p0 = bias_pool(w & 0x0F0F0F0Fu, nz);
                p1 = bias_pool((w >> 4) & 0x0F0F0F0Fu, nz);
              } else {                                           // 2-bit: 16 codes per dword
                const uint32_t w = st[half] >> (4 * jj2);        // k = 2*jj2, 2*jj2+1
                p0 = bias_pool(w & 0x03030303u, nz);
                p1 = bias_pool((w >> 2) & 0x03030303u, nz);
              }
              bfrag[2 * jj2] = p0; bfrag[2 * jj2 + 1] = p1;
            } else {
              const uint32_t mw = mk[jb];
              const uint32_t mb = jj == 0 ? (mw & 0xFFu) : __builtin_amdgcn_ubfe(mw, 8 * jj, 8);
              const uint32_t r = jj == 0 ? 0u : (uint32_t)__builtin_popcount(mw & ((1u << (8 * jj)) - 1u));
              const uint32_t w = jj == 0 ? st[0] : window<C::NW>(st, r * C::SB);
              if (C::SB == 4) {
                p0 = bias_pool(w & 0x0F0F0F0Fu, nz);
                p1 = bias_pool((w >> 4) & 0x0F0F0F0Fu, nz);
              } else {
                const uint32_t lo16 = w & 0xFFFFu;
                const uint32_t t2 = (lo16 << 14) | lo16;
                p0 = bias_pool(t2 & 0x03030303u, nz);
                p1 = bias_pool((t2 >> 4) & 0x03030303u, nz);
              }
              const uint2 sel = lut[mb * LUT_LANES + l16];
              bfrag[2 * jj2] = perm(p1, p0, sel.x);
              bfrag[2 * jj2 + 1] = perm(p1, p0, sel.y);
            }
          }
          const int t = 2 * jb + half;                            // fragment index in the chunk
          const v4i bv = (v4i){(int)bfrag[0], (int)bfrag[1], (int)bfrag[2], (int)bfrag[3]};
#pragma unroll
          for (int p = 0; p < MP; ++p) {
            const v4i av = *(const v4i*)(smem + aaddr[p] + 16 * t);
            acc[p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[p], 0, 0, 0);
#ifdef CBK_NOP_AFTER_MFMA
            asm volatile("s_nop 7\n s_nop 7" ::: "memory");
#endif
          }
          // ---- end of a quantisation group: int32 -> float, times scale * delta
          if ((C::NGC == 2 && t == 3) || t == 7) {
            const int g = (C::NGC == 2 && t == 7) ? 1 : 0;
#pragma unroll
            for (int p = 0; p < MP; ++p) {
              const int mi = 2 * p + o_mloc;
              const float* dl = delta + (mi < a.M ? mi : 0) * (NCH + 4) + 4 * S + o_s0;
              const float f0 = (float)(acc[p][0] * 256 + acc[p][1]);
              const float f1 = (float)(acc[p][2] * 256 + acc[p][3]);
              ysum[p] = fmaf(f0, sc[0][g] * dl[0], ysum[p]);
              ysum[p] = fmaf(f1, sc[1][g] * dl[1], ysum[p]);
              acc[p] = (v4i){0, 0, 0, 0};
            }
          }
        }
      }
    }
    // ---- combine the two lane quarters that hold the same activation row, then the waves
#pragma unroll
    for (int p = 0; p < MP; ++p) {
      const float v = ysum[p] + __shfl_xor(ysum[p], 16, 64);
      const int mi = 2 * p + o_mloc;
      if ((kq & 1) == 0 && mi < a.M) red[((buf * GV_WAVES + wave) * GV_MAX_M + mi) * 16 + wr] = v;
    }
    __syncthreads();
    if (tid < 16 * a.M) {
      const int mi = tid >> 4, r = tid & 15, k = tile * 16 + r;
      if (k < m.K) {
        float v = 0.f;
        const int nw = nS < GV_WAVES ? nS : GV_WAVES;
        for (int w = 0; w < nw; ++w) v += red[((buf * GV_WAVES + w) * GV_MAX_M + mi) * 16 + r];
        if (a.bias) v += (a.ydt == CBK_F32) ? ((const float*)a.bias)[k]
                       : (a.ydt == CBK_F16) ? h2f(((const uint16_t*)a.bias)[k]) : bf2f(((const uint16_t*)a.bias)[k]);
        const size_t o = (size_t)mi * a.ldy + k;
        if (a.ydt == CBK_F32) ((float*)a.y)[o] = v;
        else if (a.ydt == CBK_F16) ((uint16_t*)a.y)[o] = f2h(v);
        else ((uint16_t*)a.y)[o] = f2bf(v);
      }
    }
    buf ^= 1;
  }
}

// ------------------------------------------------------------------ host side
static size_t lds_bytes(const DMat& m, int M) {
  const int NCH = m.N / 128;
  return (size_t)LUT_BYTES + ZERO_BYTES + (size_t)M * 2 * m.N + (size_t)M * (NCH + 4) * 4 +
         (size_t)2 * GV_WAVES * GV_MAX_M * 16 * 4;
}

static bool keep_supported(int keep) { return keep == 10 || keep == 16 || keep == 23; }

bool gemv_fast_takes(const DMat& m, int M) {
  if (M < 1 || M > GV_MAX_M) return false;
  if (m.cs_rows > 1) return false;
  if (!(m.flags & CBK_FLAG_ZERO_LE_128)) return false;
  const int fam = family_of(m.layout);
  if (fam == FAM_BLK) { if (!keep_supported(m.keep)) return false; }
  else if (fam == FAM_DENSE) { if (m.bits == 8) return false; }
  else return false;
  if (m.bits != 2 && m.bits != 3 && m.bits != 4) return false;
  return (size_t)M * 2 * m.N <= (size_t)X_LDS_BUDGET;
}

size_t gemv_fast_workspace(const DMat&, int) { return 0; }

template <int BITS, int KEEP, int GRP, int MP>
static int launch_cfg(const GvArgs& a, size_t lds, hipStream_t st) {
  auto kern = gemv_mfma_kernel<BITS, KEEP, GRP, MP>;
  static std::atomic<size_t> configured{0};
  if (configured.load(std::memory_order_relaxed) < lds) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 512) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(160 * 1024, std::memory_order_relaxed);
  }
  int blocks = a.ntiles < 512 ? a.ntiles : 512;
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(GV_THREADS), lds, st, a);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

template <int BITS, int KEEP, int GRP>
static int launch_mp(const GvArgs& a, size_t lds, hipStream_t st) {
  const int mp = (a.M + 1) / 2;
  if (mp == 1) return launch_cfg<BITS, KEEP, GRP, 1>(a, lds, st);
  if (mp == 2) return launch_cfg<BITS, KEEP, GRP, 2>(a, lds, st);
  return launch_cfg<BITS, KEEP, GRP, 4>(a, lds, st);
}

template <int BITS, int KEEP>
static int launch_grp(const GvArgs& a, size_t lds, hipStream_t st) {
  return a.m.group == 64 ? launch_mp<BITS, KEEP, 64>(a, lds, st) : launch_mp<BITS, KEEP, 128>(a, lds, st);
}

template <int BITS>
static int launch_keep(const GvArgs& a, size_t lds, hipStream_t st) {
  switch (family_of(a.m.layout) == FAM_DENSE ? 0 : a.m.keep) {
    case 0: return launch_grp<BITS, 0>(a, lds, st);
    case 10: return launch_grp<BITS, 10>(a, lds, st);
    case 16: return launch_grp<BITS, 16>(a, lds, st);
    case 23: return launch_grp<BITS, 23>(a, lds, st);
    default: return CBK_ERR_UNSUPPORTED;
  }
}

int launch_gemv_fast(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                     const void* bias, void*, size_t, hipStream_t st) {
  GvArgs a;
  a.m = m; a.x = (const uint16_t*)x; a.ldx = ldx; a.M = M; a.y = y; a.ydt = ydt; a.ldy = ldy; a.bias = bias;
  a.xdt = xdt; a.ntiles = (m.K + 15) / 16;
  const size_t lds = lds_bytes(m, M);
  switch (m.bits) {
    case 2: return launch_keep<2>(a, lds, st);
    case 3: return launch_keep<3>(a, lds, st);
    case 4: return launch_keep<4>(a, lds, st);
    default: return CBK_ERR_UNSUPPORTED;
  }
}

}  // namespace cbk
