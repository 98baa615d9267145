// Decode GEMV / skinny GEMM (1 <= M <= 8) on the gfx950 int8 matrix cores.
//
// Idea.  At 8 TB/s and ~3 bits per weight the chip must consume ~20e12 weights per second,
// which leaves about two vector-ALU instructions per weight: a per-weight convert + FMA
// dequantiser cannot keep up.  So the weights stay integers.  Every lane decodes 128
// consecutive columns of ONE weight row into signed bytes (q - zero for a kept column, 0
// for a pruned one) sixteen at a time, and hands each 16-byte fragment to
// v_mfma_i32_16x16x64_i8 as the B operand.  The A operand is the activation vector in
// block fixed point: per 128-column chunk, x' = x * col_scale is written as
// delta * (65536*d2 + 256*d1 + d0) with three int8 digits (|x' - delta*X| <= max|x'| / 2^24,
// i.e. float32 resolution relative to the largest activation of the chunk).  The
// matrix core produces exact int32 dot products per (row, chunk, digit); one float FMA per
// row and quantisation group applies scale * delta.  A pruned column multiplies a literal
// zero byte, so it contributes exactly 0 whatever the zero point holds.
//
// Work decomposition.  A wavefront owns a tile of 16 weight rows; lane l works on row l%16
// and on the 128-column chunk 4*S + l/16 of macro-step S (512 columns).  The four lane
// quarters are four different quantisation groups, which one MFMA would add up; the rows of
// the A operand therefore carry (activation row, quarter, digit) variants that are non-zero
// in one quarter only, and the 16x16 result keeps the groups apart.  One persistent workgroup
// of sixteen wavefronts per CU owns a contiguous range of row tiles; a tile is cut into up
// to 16 column parts and the (tile, part) items are dealt round-robin to the wavefronts.  There
// is no barrier per tile: the partial sums of a tile meet in an LDS slot and the wavefront that
// arrives last adds them in part order, so results are run-to-run identical.
// For 2 <= M <= 8 the headline configurations put the lane quarters on the four 32-column
// blocks of one chunk instead of on four chunks (see block_split_capable below), so that
// every MFMA serves four activation rows (M = 5..8: two MFMAs per decoded fragment, one weight
// pass); sums are formed in the same order as for M = 1, so a row's result does not depend on M.
// The activation digits and the byte-permute selector table live in LDS for the whole launch;
// where the digits of all rows of a matrix do not fit (two to eight activation rows of a long
// row) they are staged one column slab at a time, whole split-K parts per slab, while the partial
// sums of the tiles wait in their LDS slots: the weights are still read once.  With room for the
// part sums in the caller's workspace such rows go to gemv_split_kernel instead, where a
// workgroup owns one column slab of a range of tiles and a second kernel adds the parts.
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
#include "cbk_decode.h"

namespace cbk {

constexpr int GV_WAVES = 16;
constexpr int GV_THREADS = GV_WAVES * 64;
#ifndef CBK_LUT_LANES
#define CBK_LUT_LANES 8
#endif
constexpr int LUT_LANES = CBK_LUT_LANES;      // lane-private copies of the selector table
constexpr int LUT_BYTES = 256 * LUT_LANES * 8;
constexpr int ZERO_BYTES = 256;
constexpr int CNT_SLOTS = 64;                 // most reduction slots (arrival counters)
constexpr int CNT_BYTES = CNT_SLOTS * 4;       // at a fixed place: zeroed before the arguments are read
constexpr int X_LDS_BUDGET = 112 * 1024;      // activation digits of one column slab: M * 3 * columns bytes (of 160 KB LDS)
constexpr int DELTA_LDS_BUDGET = 16 * 1024;   // one float per 128-column chunk and activation row (eight rows of 65024
                                              // columns; the digits take what is left: a part of 4096 columns of
                                              // eight rows, 96 KB, still fits beside 24 KB of reduction slots)
constexpr int NDIG = 3;                       // int8 digits per activation
// The digit rows of the matrix-core kernels lie X_PAD bytes further apart than their length.  The
// sixteen lanes of a quarter read sixteen bytes each from up to twelve different rows (activation
// row, digit) at the same column; row lengths are multiples of 128 bytes, and unpadded rows would
// all start in the same LDS banks.
constexpr int X_PAD = 16;
constexpr int GV_MAX_M = 8;                     // 5..8 only in the block-per-quarter arrangement
constexpr int GV_MAX_BATCH = 8;               // matrices per launch

// ------------------------------------------------------------------ kernel configuration
// MP: MFMA passes per fragment = activation rows M.
template <int BITS, int KEEP, int GRP, int MP>
struct Cfg : CodeCfg<BITS, KEEP, GRP> {};

// One matrix of a batched launch.
struct GvMat {
  DMat m;
  const uint16_t* x;       // activations [M][ldx], fp16 or bf16 bits
  int64_t ldx;
  int order;               // digit order inside a 16-column fragment: 0 column order, 1 / 2 dense
  int par;                 // 1: two col_scale vectors by row parity; activation row v of the kernel is
                           // row v / 2 of x scaled by vector v % 2, and weight row k keeps the rows v = k (mod 2)
  void* y;
  const void* bias;
  int64_t ldy;
  int ntiles;              // ceil(K / 16)
  int nS;                  // macro-steps per tile = ceil(N / 512)
  int cost0;               // sum of ntiles * nS over the matrices before this one
  int spi, sk;             // macro-steps per work item, work items per tile
  int sp;                  // parts per column slab: the activation digits of sp * spi * 512 columns are staged at a
                           // time (sp == sk: the whole row at once)
  // branch-free addressing of either byte order.  Row r of tile t starts at
  // data + t * tile_a + r * lane_mul and its 16-byte units are 1 << ush bytes apart; the scale /
  // zero entry of (row, group g) has index t * 16 * G + r * sz_mul + (g << csh).
  uint32_t tile_a, lane_mul, sz_mul;
  int ush, csh;
  // Divisions the kernel would otherwise do in software, sixteen wavefronts at a time on the one
  // scalar unit of a CU: a / nS = (a * inv_nS) >> 32 (inv_nS = 0: not exact for this launch, divide),
  // w / sp = (w * inv_sp) >> 16 for w <= 16, and 16 / sp, 16 % sp.
  uint32_t inv_nS, inv_sp;
  int dq_t, dq_p;
};

// What every wavefront needs before it can find its work: small, first in the kernel
// arguments and read in one go (each dependent read of the argument block is a round trip).
struct GvHead {
  int n, M, xdt, ydt;
  int cq, cr;              // cost units per workgroup: cq, and one more for the first cr workgroups
  int xq_cap, delta_cap;   // LDS bytes reserved for digits / floats reserved for delta
  int sk_cap, nslot, red_floats;   // reduction slots: nslot x sk_cap x M x 16 floats
  int cost_end[GV_MAX_BATCH];      // cost0 + ntiles * nS of every matrix (INT_MAX from entry n on)
};

struct GvBatch {
  GvHead h;
  GvMat mat[GV_MAX_BATCH];
};

// Column order of the activation digits inside a 16-column fragment: the byte order in which
// the decoder emits the weights.  The bitmap layouts come out in column order (the permute
// puts them there); the dense layouts skip the permute and come out as the spread leaves them.
__host__ __device__ constexpr int frag_col(int bits, bool dense, int bi) {
  if (!dense) return bi;
  if (bits == 2) return (bi >> 2) + 4 * (bi & 3);                                 // byte 4k+j <- column k+4j
  return ((bi >> 3) << 3) + 2 * (bi & 3) + ((bi >> 2) & 1);                       // even | odd per 8
}

// Two ways to lay a macro-step (16 rows x 512 columns) on the 16x16x64 MFMA.
//  * quarter-per-chunk: lane quarter kq decodes chunk 4S + kq; one MFMA adds four different
//    quantisation groups, so the A rows are (quarter, digit) and one activation row needs one
//    pass.  Used for M = 1 and for every configuration below that cannot use the other way.
//  * quarter-per-block: lane quarter kq decodes block kq (32 columns) of each of the four
//    chunks; one MFMA covers 64 columns of a single group, the A rows are (activation row,
//    digit), and up to four activation rows share every MFMA.  Needs group 128 and a block's
//    code bits to be 4, 8 or 16 whole bytes.
__host__ __device__ constexpr bool block_split_capable(int bits, int keep, int grp) {
  const int cb = (keep == 0 ? 32 : keep) * bits;
  return grp == 128 && bits != 3 && (cb == 32 || cb == 64 || cb == 128);
}

// ------------------------------------------------------------------ activation prep
// x' = x * col_scale per 128-column chunk -> delta and three signed int8 digits per column:
// x' ~= delta * (65536*d2 + 256*d1 + d0),  delta = max|x'| / (127 * 65536).  Every workgroup
// converts the activations it needs into its own LDS (a few hundred instructions per thread,
// overlapped with the first weight loads).  One thread converts 16 columns at a time; the
// eight threads of a chunk agree on its maximum with three lane exchanges.
struct XLoad { uint4 x[2], c[2]; };

// global loads of staging item `it` of the column slab that starts at column col0 and is n16 * 16
// columns wide (activation row it / n16, columns col0 + 16 * (it % n16) ...)
__device__ inline void stage_load(const uint16_t* x, int64_t ldx, const uint16_t* cs, int N, int col0, int n16, int it,
                                  bool one_row, int par, XLoad& r) {
  const int row = one_row ? 0 : it / n16, c16 = it - row * n16;
  const int xrow = par ? row >> 1 : row;
  const uint16_t* xp = x + (size_t)xrow * ldx + col0 + c16 * 16;
  r.x[0] = ((const uint4*)xp)[0]; r.x[1] = ((const uint4*)xp)[1];
  r.c[0] = make_uint4(0, 0, 0, 0); r.c[1] = make_uint4(0, 0, 0, 0);
  if (cs) {
    const uint16_t* cp = cs + (par ? (size_t)(row & 1) * N : (size_t)0) + col0 + c16 * 16;
    r.c[0] = ((const uint4*)cp)[0]; r.c[1] = ((const uint4*)cp)[1];
  }
}

// conversion of one loaded item into digits and delta in LDS; the eight consecutive lanes of a
// chunk are always active together (the item count is a multiple of 8)
// (digits at row stride Ns = 16 * n16 + pad bytes, deltas at the chunk's index in the whole row: ch0 is
// the slab's first chunk)
template <int ORDER>
__device__ inline void stage_convert(const XLoad& r, bool has_cs, int xdt, int N, int ch0, int n16, int it, bool one_row,
                                     int8_t* xq, float* delta, int pad = 0) {
  const int NCH = N >> 7, Ns = n16 * 16 + pad;
  const int row = one_row ? 0 : it / n16, c16 = it - row * n16;
  const uint32_t* xw = (const uint32_t*)r.x;
  const uint32_t* cw = (const uint32_t*)r.c;
  float xv[16];
  if (xdt == CBK_F16) {                                            // one uniform branch, not one per element
#pragma unroll
    for (int e = 0; e < 16; ++e) xv[e] = h2f((uint16_t)(xw[e >> 1] >> (16 * (e & 1))));
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e) xv[e] = bf2f((uint16_t)(xw[e >> 1] >> (16 * (e & 1))));
  }
  if (has_cs) {
#pragma unroll
    for (int e = 0; e < 16; ++e) xv[e] *= h2f((uint16_t)(cw[e >> 1] >> (16 * (e & 1))));
  }
  float mx = 0.f;
#pragma unroll
  for (int e = 0; e < 16; ++e) mx = fmaxf(mx, fabsf(xv[e]));
  // maximum over the eight lanes of the chunk with register-to-register lane moves: swap
  // neighbours, swap pairs, mirror the eight-lane half row (every lane of a quad holds the
  // quad's maximum by then, so the mirror image is the other quad's)
  mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, mx), 0xB1, 0xF, 0xF, true)));
  mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, mx), 0x4E, 0xF, 0xF, true)));
  mx = fmaxf(mx, __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, mx), 0x141, 0xF, 0xF, true)));
  // delta = max|x'| / 8323072 (= 127 * 65536: 24 signed bits) by a multiplication, its reciprocal by the
  // hardware approximation and one Newton step; two divisions were a tenth of this function.
  // (24 bits, not 23 with a cheaper rounding: activations of 1e4 at the pruned columns of a chunk,
  // the reference's own probe, leave the ordinary ones 10 bits less, and the result must still
  // meet the layer tolerance.)
  const float d = mx > 1e-30f ? mx * (1.f / 8323072.f) : 1.f;
  float inv = __builtin_amdgcn_rcpf(d);
  inv = inv * fmaf(-d, inv, 2.f);
  // X + 0x808080 has the bytes d0 + 128, d1 + 128, d2 + 128 of the balanced base-256 digits
  // (X = d0 + 256 d1 + 65536 d2, -128 <= d < 128), so the digits of four columns are byte
  // permutes of the four biased integers and one xor per digit plane
  uint32_t dw[NDIG][4];
  uint32_t xb[16];
#pragma unroll
  for (int bi = 0; bi < 16; ++bi) {
    const float v = ORDER == 0 ? xv[bi] : ORDER == 1 ? xv[frag_col(4, true, bi)] : xv[frag_col(2, true, bi)];
    xb[bi] = (uint32_t)((int)rintf(v * inv) + 0x808080);          // |X| <= 127 * 65536 (+ 2 from the rounding of inv)
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t a = perm(xb[4 * q + 1], xb[4 * q], 0x05010400u);       // d0 d0 d1 d1 of columns 0, 1
    const uint32_t b = perm(xb[4 * q + 3], xb[4 * q + 2], 0x05010400u);   // and of columns 2, 3
    const uint32_t c01 = perm(xb[4 * q + 1], xb[4 * q], 0x0C0C0602u);     // d2 d2 0 0
    const uint32_t c23 = perm(xb[4 * q + 3], xb[4 * q + 2], 0x06020C0Cu); // 0 0 d2 d2
    dw[0][q] = (c01 | c23) ^ 0x80808080u;
    dw[1][q] = perm(b, a, 0x07060302u) ^ 0x80808080u;
    dw[2][q] = perm(b, a, 0x05040100u) ^ 0x80808080u;
  }
#pragma unroll
  for (int k = 0; k < NDIG; ++k)
    *(uint4*)(xq + ((size_t)row * NDIG + k) * Ns + c16 * 16) = make_uint4(dw[k][0], dw[k][1], dw[k][2], dw[k][3]);
  if ((c16 & 7) == 0) delta[row * (NCH + 4) + ch0 + (c16 >> 3)] = d;
  if (ch0 == 0 && c16 < 4) delta[row * (NCH + 4) + NCH + c16] = 0.f;   // chunks past N
}

// y(l) + y(l ^ 16), then that + the same of lane l ^ 32: the sum over the four lane quarters, in
// every lane, with the two row-swap instructions of gfx950 instead of two trips through the LDS
// crossbar.  (Through inline assembly: the compiler's builtin for the swaps returned the same
// register for both results.)  The s_nop covers the wait states between a VALU write and the swap.
__device__ inline float quarter_sum(float y) {
  float a = y, b = y;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  const float t = a + b;
  float c = t, d = t;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(c), "+v"(d));
  return c + d;
}

// Sum over the wavefront, in every lane, without a trip through LDS: quads, half rows and rows by
// DPP lane moves (each step adds the mirror image that holds the other half's sum), then the four
// rows with the swap instructions.
__device__ inline float wave_sum_dpp(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));    // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));    // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));   // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));   // row_mirror
  return quarter_sum(v);
}

// ------------------------------------------------------------------ one 32-column block
// mask bytes of a block and the number of survivors before each of them
template <class C>
__device__ inline void split_mask(uint32_t mw, uint32_t (&mb)[4], uint32_t (&rk)[4]) {
  if (!C::DENSE) {
    mb[0] = mw & 0xFFu; mb[1] = __builtin_amdgcn_ubfe(mw, 8, 8); mb[2] = __builtin_amdgcn_ubfe(mw, 16, 8); mb[3] = mw >> 24;
    rk[0] = 0; rk[1] = (uint32_t)__builtin_popcount(mb[0]);
    rk[2] = rk[1] + (uint32_t)__builtin_popcount(mb[1]); rk[3] = rk[2] + (uint32_t)__builtin_popcount(mb[2]);
  }
}

// ranks and table reads of one block
template <class C>
__device__ inline void fetch_selectors(uint32_t mw, const uint2* lut, uint32_t l16, uint32_t (&rk)[4], uint2 (&sel4)[4]) {
  uint32_t mb[4];
  split_mask<C>(mw, mb, rk);
  if (!C::DENSE) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) sel4[jj] = lut[mb[jj] * LUT_LANES + l16];
  }
}

// Sixteen columns (half `half` of the block whose code stream is st) as signed bytes q - zero,
// pruned columns 0: the B operand of one MFMA.
// sel4: the selectors of the block's four mask bytes, read from the table by fetch_selectors.
template <class C, int BITS>
__device__ inline void decode_half(const uint32_t (&st)[C::NW], const uint32_t (&rk)[4], const uint2 (&sel4)[4],
                                   uint32_t nz, int half, uint32_t (&bfrag)[4], uint32_t hw = 0) {
#pragma unroll
  for (int jj2 = 0; jj2 < 2; ++jj2) {
    const int jj = 2 * half + jj2;                       // mask byte inside the block
    uint32_t p0, p1;
    if (C::DENSE) {
      if (C::SB == 4) {
        const uint32_t w = st[jj];
        p0 = bias_pool(w & 0x0F0F0F0Fu, nz);
        p1 = bias_pool((w >> 4) & 0x0F0F0F0Fu, nz);
      } else {                                           // 2-bit: 16 codes per dword
        const uint32_t w = st[half] >> (4 * jj2);
        p0 = bias_pool(w & 0x03030303u, nz);
        p1 = bias_pool((w >> 2) & 0x03030303u, nz);
      }
      bfrag[2 * jj2] = p0; bfrag[2 * jj2 + 1] = p1;
    } else {
      uint32_t w;
      if (jj == 0) w = st[0];
      else w = window<C::NW>(st, rk[jj] * C::SB);
      if (C::HI2) {
        uint32_t h0, h1;
        hi2_pools(hw, jj == 0 ? 0u : rk[jj], h0, h1);
        p0 = bias_pool((w & 0x0F0F0F0Fu) | h0, nz);
        p1 = bias_pool(((w >> 4) & 0x0F0F0F0Fu) | h1, nz);
      } else if (C::SB == 4) {
        p0 = bias_pool(w & 0x0F0F0F0Fu, nz);
        p1 = bias_pool((w >> 4) & 0x0F0F0F0Fu, nz);
      } else {
        const uint32_t lo16 = w & 0xFFFFu;
        const uint32_t t2 = (lo16 << 14) | lo16;
        p0 = bias_pool(t2 & 0x03030303u, nz);
        p1 = bias_pool((t2 >> 4) & 0x03030303u, nz);
      }
      const uint2 sel = sel4[jj];
      bfrag[2 * jj2] = perm(p1, p0, sel.x);
      bfrag[2 * jj2 + 1] = perm(p1, p0, sel.y);
    }
  }
}

// ------------------------------------------------------------------ the decode kernel
template <class C>
struct Loads {
  uint32_t mk[4];
  uint32_t raw[C::NL];
  uint32_t zraw;
  uint32_t sc[C::NGC];        // fp16 bits of the scales of this lane's chunk
  uint32_t h2[C::HI2 ? 4 : 1];   // BLK1632_6: the chunk's four dwords of high bits
};

template <int BITS, int KEEP, int GRP, int MP>
__global__ __launch_bounds__(GV_THREADS) void gemv_mfma_kernel(GvBatch b) {
  using C = Cfg<BITS, KEEP, GRP, MP>;
  constexpr bool QB = (MP == 4 || MP == 8) && block_split_capable(BITS, KEEP, GRP);
  constexpr int NG = MP == 8 ? 2 : 1;                  // groups of four activation rows, one MFMA each per fragment
  static_assert(MP <= 4 || QB, "more than four activation rows need the block-per-quarter arrangement");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // in a scalar register: positions are scalar work
  uint2* lut = (uint2*)smem;
  uint8_t* zreg = smem + LUT_BYTES;
  int* cnt = (int*)(zreg + ZERO_BYTES);                // [CNT_SLOTS] arrival counters
  int8_t* xq = (int8_t*)cnt + CNT_BYTES;
  // The argument block is read in two dependent steps (header, then the record of the first
  // matrix), each a round trip to memory for the first wavefronts that ask.  Touch its first
  // cache lines now, with scalar loads whose results nobody uses, so that both steps find them
  // in the scalar cache; the registers stay reserved until the loads have returned.
  uint32_t ka[5];
  static_assert(sizeof(GvBatch) >= 0x104, "the five touched lines lie inside the argument block");
  {
    const auto kp = __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("s_load_dword %0, %5, 0x0\n\ts_load_dword %1, %5, 0x40\n\ts_load_dword %2, %5, 0x80\n\t"
                 "s_load_dword %3, %5, 0xc0\n\ts_load_dword %4, %5, 0x100"
                 : "=&s"(ka[0]), "=&s"(ka[1]), "=&s"(ka[2]), "=&s"(ka[3]), "=&s"(ka[4]) : "s"(kp));
  }
  // Selector table, zero row and counters do not depend on the arguments: they are written
  // while the argument block is on its way, and published by the barrier that follows the
  // staging of the first matrix's activations (nothing reads them before).
  {
    using C0 = Cfg<BITS, KEEP, GRP, MP>;
    if (tid < 256) {
      const uint2 e = make_selectors((uint32_t)tid, C0::SEL_KIND);
#pragma unroll
      for (int j = 0; j < LUT_LANES; ++j) lut[tid * LUT_LANES + j] = e;
    } else if (tid < 256 + ZERO_BYTES / 4) {
      ((uint32_t*)zreg)[tid - 256] = 0u;
    } else if (tid < 256 + ZERO_BYTES / 4 + CNT_SLOTS) {
      cnt[tid - 256 - ZERO_BYTES / 4] = 0;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::"s"(ka[0]), "s"(ka[1]), "s"(ka[2]), "s"(ka[3]), "s"(ka[4]));
  }
  const GvHead h = b.h;
  float* delta = (float*)(xq + h.xq_cap);
  float* red = delta + h.delta_cap;                    // [nslot][sk_cap][M][16] partial sums

  const int wr = lane & 15, kq = lane >> 4;            // weight row in tile / lane quarter
  const uint32_t l16 = lane & (LUT_LANES - 1);
  // role of this lane's row in the A operand: variant i = lane%16 = 4 * quarter + digit
  // (digit 3 is an all-zero row); in the result, lane quarter kq holds the three digit sums
  // of its own chunk, so every lane post-processes exactly the chunk it decoded
  const int a_slice = wr >> 2, a_dig = wr & 3;
  const uint32_t xq_off = (uint32_t)((uint8_t*)xq - smem), z_off = (uint32_t)(zreg - smem);

  // the tiles of this workgroup: those whose first cost unit falls in [c0, c1)
  const int bx = (int)blockIdx.x;
  const int c0 = bx * h.cq + (bx < h.cr ? bx : h.cr);
  const int c1 = c0 + h.cq + (bx < h.cr ? 1 : 0);
  bool first = true;
  // first matrix with cost units at or after c0
  int mi0 = 0;
#pragma unroll
  for (int i = 0; i < GV_MAX_BATCH - 1; ++i) mi0 += h.cost_end[i] <= c0 ? 1 : 0;     // (entries past n never count)

  // The first record is requested together with the header: most workgroups start with it, and
  // for them the second round trip through the argument block before any load goes out is gone.
  // One trip of the loop below = one matrix, or, for a matrix whose rows are longer than the
  // staging area (more than one activation row only), one column slab of one group of its tiles.
  // A single loop level on purpose: nested loops made the compiler keep several dozen more
  // scalars alive across the decode loop, spilled into vector registers.
  constexpr bool SLABS = MP > 1;
  GvMat gm = b.mat[0];
  int g_lo = -1, pa = 0;                                          // tile group and first part of the next trip
  for (int mi = mi0; mi < h.n;) {
    if (mi != 0) gm = b.mat[mi];                                  // one read of the whole record
    if (gm.cost0 >= c1) break;                                    // uniform over the workgroup
    const DMat& m = gm.m;
    const int nS = gm.nS;
    const int N = m.N, NCH = N >> 7;
    // items: tile tl (local), part j of SK; part j covers macro-steps [j*spi, min(nS,(j+1)*spi))
    const int SK = gm.sk, spi = gm.spi, SP = SLABS ? gm.sp : SK;
    const int pn = SLABS && SK - pa >= SP ? SP : SK - pa;         // parts of this slab
    const int col0 = SLABS ? pa * spi * 512 : 0;                  // its columns: [col0, col0 + Ns)
    const int Ns = SLABS && N - col0 >= pn * spi * 512 ? pn * spi * 512 : N - col0;
    const int ch0 = col0 >> 7;

    // The activation loads go out first, as soon as the matrix is known: before the weight loads,
    // because the weight prefetch of a whole launch is tens of megabytes and a request queued
    // behind it would keep every wavefront from decoding until that burst has drained; and before
    // the rest of the set-up, which is a few hundred scalar instructions on the one scalar unit
    // the sixteen wavefronts share.
    const int n16 = Ns >> 4, xitems = h.M * n16;                  // a multiple of 8
    // The first two items of a thread (all there are, but for the longest rows) are loaded here
    // and converted outside the loop further down: inside it the compiler's wait for an item's
    // loads has to allow for the trip in which they were issued after the weight loads, and so
    // waits for the weight loads as well; the conversion would start only once the first weights
    // have arrived instead of running while they are on their way.
    // (The second item only where its sixteen registers do not push the kernel into scratch.)
    constexpr bool PRE2 = MP == 1 || (MP == 4 && QB);
    int xit = tid;
    XLoad xl, xl2;
    if (xit < xitems) stage_load(gm.x, gm.ldx, m.cs, N, col0, n16, xit, MP == 1, gm.par, xl);
    if (PRE2 && xit + GV_THREADS < xitems)
      stage_load(gm.x, gm.ldx, m.cs, N, col0, n16, xit + GV_THREADS, MP == 1, gm.par, xl2);
    __builtin_amdgcn_sched_barrier(0);

    // ceil((c - cost0) / nS), 0 for c <= cost0
    auto tiles_before = [&](int c) -> int {
      const int a = c - gm.cost0 + nS - 1;
      if (a < nS) return 0;
      return gm.inv_nS ? (int)__umulhi((uint32_t)a, gm.inv_nS) : a / nS;
    };
    int T_lo = tiles_before(c0), T_hi = tiles_before(c1);
    T_hi = T_hi > gm.ntiles ? gm.ntiles : T_hi;
    if (T_lo >= T_hi) { ++mi; continue; }                         // uniform over the workgroup
    // A row whose digits do not fit in LDS is staged and multiplied slab by slab (SP parts of
    // every tile at a time).  A tile's partial sums then wait in their reduction slot across the
    // slabs, so the tiles are taken nslot at a time and the slots are never reused inside a group.
    const bool slabbed = SLABS && SP < SK;
    const int gt = h.nslot >> 1;                                  // tiles per barrier group, a power of two
    const int gsh = slabbed ? 30 : 31 - __builtin_clz((unsigned)gt);   // its logarithm: no division per item
    const int tgs = slabbed ? h.nslot : T_hi - T_lo;              // tiles per pass over the slabs

    // matrix constants, read from the kernel arguments once
    const uint8_t* const m_data = m.data;
    const uint16_t* const m_scale = m.scale;
    const uint8_t* const m_zero = m.zero;
    const int m_K = m.K, m_G = m.G, ush = gm.ush, csh = gm.csh;
    const uint32_t tile_a = gm.tile_a, lane_mul = gm.lane_mul, sz_mul = gm.sz_mul, code_u0 = m.code_off >> 4;
    const int last_S = nS - 1;
    const int t_lo = SLABS && g_lo >= 0 ? g_lo : T_lo;
    const int t_hi = SLABS && t_lo + tgs < T_hi ? t_lo + tgs : T_hi;
    const int last_tile = t_hi - 1;

    // ---- issue the loads of one (tile, macro-step) position; out-of-range positions are clamped
    // Everything that depends only on (tile, S) is scalar work; a lane adds a 32-bit offset.
    auto issue = [&](int tile, int S, Loads<C>& L) {
      tile = tile < last_tile ? tile : last_tile;
      S = S < last_S ? S : last_S;
      const int S4 = 4 * S;
      const int rlim = m_K - 1 - tile * 16;                         // rows past K repeat row K - 1
      const uint32_t wrc = (uint32_t)(wr < rlim ? wr : rlim);
      const uint32_t lane_off = __umul24(wrc, lane_mul);
      const int klim = NCH - 1 - S4;                                // chunks past N repeat chunk NCH - 1
      const uint32_t chl = (uint32_t)(kq < klim ? kq : klim);
      // Every address is one of the matrix's three base pointers plus a 32-bit offset (the host
      // admits only matrices whose arrays are smaller than 4 GB): a scalar part that depends on
      // (tile, S) and a lane part; one add per load, no 64-bit arithmetic per step.
      const uint32_t so_t = (uint32_t)tile * tile_a;                 // scalar: start of the tile's rows
      const uint32_t so_g = (uint32_t)tile * (uint32_t)(16 * m_G);   // scalar: first scale / zero of the tile
      if constexpr (QB) {
        // block kq of the chunks 4S .. 4S+3: one mask dword and CB / 8 code bytes each
        constexpr uint32_t BB = C::CB / 8;
        const uint32_t voff_m = lane_off + (uint32_t)kq * 4u;
        const uint32_t voff_c = lane_off + ((((uint32_t)kq * BB) >> 4) << ush) + (((uint32_t)kq * BB) & 15u);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          int chc = S4 + c;
          chc = chc < NCH ? chc : NCH - 1;
          if (!C::DENSE) L.mk[c] = *(const uint32_t*)(m_data + (so_t + ((uint32_t)chc << ush) + voff_m));
          const uint8_t* cp = m_data + (so_t + ((code_u0 + (uint32_t)chc * (C::CHB / 128)) << ush) + voff_c);
          if (C::CB == 32) {
            L.raw[c] = *(const uint32_t*)cp;
          } else if (C::CB == 64) {
            const uint2 v = *(const uint2*)cp;
            L.raw[2 * c] = v.x; L.raw[2 * c + 1] = v.y;
          } else {
            const uint4 v = *(const uint4*)cp;
            L.raw[4 * c] = v.x; L.raw[4 * c + 1] = v.y; L.raw[4 * c + 2] = v.z; L.raw[4 * c + 3] = v.w;
          }
        }
        // zero point and scale of group 4S + kq; the other quarters fetch them from this lane
        const uint32_t gv = so_g + ((uint32_t)S4 << csh) + __umul24(wrc, sz_mul) + (chl << csh);
        L.zraw = (uint32_t)m_zero[gv] | ((uint32_t)m_scale[gv] << 8);
        return;
      }
      const uint32_t so_s = so_t + ((uint32_t)S4 << ush);            // scalar: unit 4S of the rows
      if (!C::DENSE) {
        const uint4 v = *(const uint4*)(m_data + (so_s + lane_off + (chl << ush)));
        L.mk[0] = v.x; L.mk[1] = v.y; L.mk[2] = v.z; L.mk[3] = v.w;
      }
      // code bits of the chunk: bit ch*CHB of the code plane, fetched as whole 16-byte units
      if (C::VEC16) {
        const uint32_t so_c = so_t + ((code_u0 + (uint32_t)S4 * (C::CHB / 128)) << ush);
        const uint32_t voff = lane_off + ((chl * (C::CHB / 128)) << ush);
#pragma unroll
        for (int i = 0; i < C::NL / 4; ++i) {
          const uint4 v = *(const uint4*)(m_data + (so_c + ((uint32_t)i << ush) + voff));
          L.raw[4 * i] = v.x; L.raw[4 * i + 1] = v.y; L.raw[4 * i + 2] = v.z; L.raw[4 * i + 3] = v.w;
        }
      } else {
        const uint32_t u = (((uint32_t)S4 + chl) * (uint32_t)C::CHB) >> 7;
        const uint32_t voff = lane_off + (u << ush);
#pragma unroll
        for (int i = 0; i < C::NL / 4; ++i) {
          const uint4 v = *(const uint4*)(m_data + (so_t + ((code_u0 + (uint32_t)i) << ush) + voff));
          L.raw[4 * i] = v.x; L.raw[4 * i + 1] = v.y; L.raw[4 * i + 2] = v.z; L.raw[4 * i + 3] = v.w;
        }
      }
      if (C::HI2) {                                                 // unit ch of the plane behind mask and nibbles
        const uint4 v = *(const uint4*)(m_data + (so_t + ((3u * (uint32_t)NCH + (uint32_t)S4 + chl) << ush) + lane_off));
        L.h2[0] = v.x; L.h2[1] = v.y; L.h2[2] = v.z; L.h2[3] = v.w;
      }
      const uint32_t gv = so_g + ((uint32_t)(S4 * C::NGC) << csh) + __umul24(wrc, sz_mul) + ((chl * C::NGC) << csh);
      if (C::NGC == 1) {
        L.zraw = m_zero[gv];
        L.sc[0] = m_scale[gv];
      } else {
        const uint32_t gv1 = gv + (1u << csh);
        L.zraw = (uint32_t)m_zero[gv] | ((uint32_t)m_zero[gv1] << 8);
        L.sc[0] = m_scale[gv];
        L.sc[C::NGC - 1] = m_scale[gv1];
      }
    };

    // this wave's sequence of (tile, part, macro-step) positions: items wave, wave + 16, ...
    // (taking the later items from a shared counter instead was measured: no faster at one step
    // of loads in flight, slower on large launches)
    struct Pos { int tl, part, S; };
    const int ntl = t_hi - t_lo;
    const bool whole = !SLABS || pn == SP;                        // (a shorter last slab divides in software)
    const int dq_t = whole ? gm.dq_t : GV_WAVES / pn, dq_p = whole ? gm.dq_p : GV_WAVES % pn;
    const int w_t = whole ? (int)(((uint32_t)wave * gm.inv_sp) >> 16) : wave / pn, w_p = wave - w_t * pn;
    auto advance = [&](Pos& p) -> bool {                           // false past the last position
      const int s_end = (p.part * spi + spi < nS) ? p.part * spi + spi : nS;
      if (p.S + 1 < s_end) { ++p.S; return true; }
      p.tl += dq_t; p.part += dq_p;
      if (p.part >= pa + pn) { p.part -= pn; ++p.tl; }
      p.S = p.part * spi;
      return p.tl < ntl;
    };
    Pos p0{w_t, pa + w_p, (pa + w_p) * spi};
    bool v0 = p0.tl < ntl;
    // Two load buffers swap roles (being decoded, being loaded) by name: copying a buffer would
    // wait for the loads that are still filling it.  One step of loads in flight per wavefront
    // is the measured optimum (sixteen wavefronts per CU already cover the latency; a second
    // step in flight made the Mistral layer set 8 % slower).
    Loads<C> LA, LB;
    issue(t_lo + p0.tl, p0.S, LA);
    __builtin_amdgcn_sched_barrier(0);                            // (the first loads leave before the rest of the set-up)
    Pos p1 = p0; bool v1 = v0 && advance(p1);

    // ---- stage: selector table and counters (once), activation digits and deltas of this matrix
    if (!first) __syncthreads();                                  // previous matrix fully consumed
    first = false;
    constexpr int XORD = !C::DENSE ? 0 : (BITS == 2 ? 2 : 1);
    if (xit < xitems) stage_convert<XORD>(xl, m.cs != nullptr, h.xdt, N, ch0, n16, xit, MP == 1, xq, delta, X_PAD);
    if (PRE2 && xit + GV_THREADS < xitems)
      stage_convert<XORD>(xl2, m.cs != nullptr, h.xdt, N, ch0, n16, xit + GV_THREADS, MP == 1, xq, delta, X_PAD);
    for (xit += (PRE2 ? 2 : 1) * GV_THREADS; xit < xitems; xit += GV_THREADS) {
      stage_load(gm.x, gm.ldx, m.cs, N, col0, n16, xit, MP == 1, gm.par, xl);
      stage_convert<XORD>(xl, m.cs != nullptr, h.xdt, N, ch0, n16, xit, MP == 1, xq, delta, X_PAD);
    }
    __syncthreads();

    int bars = 0;                                                 // group barriers passed so far
    float ysum[MP];
    auto do_step = [&](Loads<C>& cur, Loads<C>& tgt) {             // decode `cur`, load the next step into `tgt`
      const int tl = p0.tl, part = p0.part, S = p0.S;
      const int tile = t_lo + tl;
      const int s_end = (part * spi + spi < nS) ? part * spi + spi : nS;
      if (S == part * spi) {                                      // first step of an item
        // slots of tile group g are reused by group g + 2: wait until group g - 1 is complete
        for (const int g = tl >> gsh; bars < g; ++bars) __syncthreads();
#pragma unroll
        for (int p = 0; p < MP; ++p) ysum[p] = 0.f;
      }
      // (unconditional: past the last position the loads repeat it; under a wave-uniform branch
      // the compiler no longer spreads them over the decode, and every launch was 2-6 % slower)
      issue(t_lo + p1.tl, p1.S, tgt);
      if constexpr (QB) {
        const int a_m = wr >> 2;                                    // activation row of this lane's A row
        uint32_t zs[4];                                             // zero | scale << 8 of the groups 4S .. 4S+3
#pragma unroll
        for (int c = 0; c < 4; ++c) zs[c] = (uint32_t)__shfl((int)cur.zraw, wr + 16 * c, 64);
        // row group g holds activation rows 4g .. 4g+3: its A operand, and in the result lane
        // quarter kq the three digit sums of activation row 4g + kq
        bool a_on[NG];
        uint32_t a_base[NG];
        int dm[NG];                                                 // the activation rows this quarter sums
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          a_on[g] = a_dig < NDIG && a_m + 4 * g < h.M;
          a_base[g] = xq_off + (uint32_t)(((a_m + 4 * g) * NDIG + a_dig) * (Ns + X_PAD) + kq * 32);
          dm[g] = kq + 4 * g < h.M ? kq + 4 * g : 0;
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int chunk = 4 * S + c;
          uint32_t aaddr[NG];
#pragma unroll
          for (int g = 0; g < NG; ++g) aaddr[g] = (a_on[g] && chunk < NCH) ? a_base[g] + (uint32_t)(chunk - ch0) * 128u : z_off;
          uint32_t rkc[4];
          uint2 selc[4];
          fetch_selectors<C>(cur.mk[c], lut, l16, rkc, selc);
          uint32_t st[C::NW];
#pragma unroll
          for (int k = 0; k < C::NW; ++k) st[k] = cur.raw[c * C::NW + k];
          const uint32_t z = zs[c] & 0xFFu;
          const uint32_t nz = 0x80808080u - z * 0x01010101u;
          v4i acc[NG];
#pragma unroll
          for (int g = 0; g < NG; ++g) acc[g] = (v4i){0, 0, 0, 0};
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            uint32_t bfrag[4];
            decode_half<C, BITS>(st, rkc, selc, nz, half, bfrag);
            const v4i bv = (v4i){(int)bfrag[0], (int)bfrag[1], (int)bfrag[2], (int)bfrag[3]};
#pragma unroll
            for (int g = 0; g < NG; ++g) {
              const v4i av = *(const v4i*)(smem + aaddr[g] + 16 * half);
              acc[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[g], 0, 0, 0);
              asm("s_nop 1" : "+v"(acc[g]));                        // see the other decode path
            }
          }
          // the 128 columns of group `chunk` are complete: rows 4 kq .. 4 kq + 2 of the result
          // are the three digit sums of activation row 4g + kq
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            const float dl = delta[dm[g] * (NCH + 4) + chunk];      // 0 past the last chunk
            const float f = fmaf((float)(acc[g][0] * 256 + acc[g][1]), 256.f, (float)acc[g][2]);
            ysum[4 * g + c] = fmaf(f, h2f((uint16_t)(zs[c] >> 8)) * dl, ysum[4 * g + c]);
          }
        }
      } else
      {
        const int chunk = 4 * S + kq;
        const bool valid = chunk < NCH;
        uint32_t aaddr[MP];
#pragma unroll
        for (int p = 0; p < MP; ++p) {
          const bool on = valid && a_slice == kq && a_dig < NDIG && p < h.M;
          aaddr[p] = on ? xq_off + (uint32_t)((p * NDIG + a_dig) * (Ns + X_PAD) + (chunk - ch0) * 128) : z_off;
        }
        // ---- bring the chunk's first code bit to bit 0 of cw[0]
        uint32_t cw[C::ND];
        align_chunk_codes<C>(cur.raw, (uint32_t)(valid ? chunk : NCH - 1), cw);

        v4i acc[MP];
#pragma unroll
        for (int p = 0; p < MP; ++p) acc[p] = (v4i){0, 0, 0, 0};

#pragma unroll
        for (int jb = 0; jb < 4; ++jb) {
          uint32_t rkc[4];
          uint2 selc[4];
          fetch_selectors<C>(cur.mk[jb], lut, l16, rkc, selc);
          uint32_t st[C::NW];                                     // code stream of block jb
          block_stream<C, BITS>(cw, jb, st);
          const uint32_t z = (C::NGC == 1) ? cur.zraw : ((cur.zraw >> (8 * (jb >> 1))) & 0xFFu);
          const uint32_t nz = 0x80808080u - z * 0x01010101u;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const int t = 2 * jb + half;                            // fragment index in the chunk
            uint32_t bfrag[4];
            decode_half<C, BITS>(st, rkc, selc, nz, half, bfrag, C::HI2 ? cur.h2[C::HI2 ? jb : 0] : 0u);
            const v4i bv = (v4i){(int)bfrag[0], (int)bfrag[1], (int)bfrag[2], (int)bfrag[3]};
#pragma unroll
            for (int p = 0; p < MP; ++p) {
              const v4i av = *(const v4i*)(smem + aaddr[p] + 16 * t);
              acc[p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[p], 0, 0, 0);
              // One idle issue slot after every MFMA.  Without it some instantiations of this
              // kernel (register allocations in which the accumulator chain changes registers)
              // returned run-to-run different sums on gfx950; with it every configuration is exact.
              asm("s_nop 1" : "+v"(acc[p]));
            }
            // ---- end of a quantisation group: int32 -> float, times scale * delta
            if ((C::NGC == 2 && t == 3) || t == 7) {
              const int g = (C::NGC == 2 && t == 7) ? 1 : 0;
#pragma unroll
              for (int p = 0; p < MP; ++p) {
                const float dl = delta[(p < h.M ? p : 0) * (NCH + 4) + chunk];      // 0 past the last chunk
                const float f = fmaf((float)(acc[p][0] * 256 + acc[p][1]), 256.f, (float)acc[p][2]);
                ysum[p] = fmaf(f, h2f((uint16_t)cur.sc[g]) * dl, ysum[p]);
                acc[p] = (v4i){0, 0, 0, 0};
              }
            }
          }
        }
      }
      if (S + 1 == s_end) {
      // ---- the item is done: add the four lane quarters (the four chunks of every macro-step)
      float part_sum[MP];
#pragma unroll
      for (int p = 0; p < MP; ++p) {
        // quarter kq holds activation row kq, one running sum per chunk position; added in the
        // order of the other decode path, so a row's result does not depend on M
        if (QB) {                                                   // (p: row group; only p < NG is used)
          const int q = p < NG ? 4 * p : 0;
          part_sum[p] = (ysum[q] + ysum[q + 1]) + (ysum[q + 2] + ysum[q + 3]);
          continue;
        }
        part_sum[p] = quarter_sum(ysum[p]);
      }
      auto store = [&](int om, int r, float v) {
        const int k = tile * 16 + r;
        if (k >= m.K) return;
        if (gm.par) {                                             // the sum scaled for the other parity is dropped
          if ((om ^ k) & 1) return;
          om >>= 1;
        }
        if (gm.bias) v += (h.ydt == CBK_F32) ? ((const float*)gm.bias)[k]
                        : (h.ydt == CBK_F16) ? h2f(((const uint16_t*)gm.bias)[k]) : bf2f(((const uint16_t*)gm.bias)[k]);
        const size_t o = (size_t)om * gm.ldy + k;
        if (h.ydt == CBK_F32) ((float*)gm.y)[o] = v;
        else if (h.ydt == CBK_F16) ((uint16_t*)gm.y)[o] = f2h(v);
        else ((uint16_t*)gm.y)[o] = f2bf(v);
      };
      if (SK == 1) {
        if (QB) {
#pragma unroll
          for (int g = 0; g < NG; ++g)
            if (kq + 4 * g < h.M) store(kq + 4 * g, wr, part_sum[g]);
        } else {
#pragma unroll
          for (int p = 0; p < MP; ++p)
            if (kq == 0 && p < h.M) store(p, wr, part_sum[p]);
        }
      } else {
        // partial sums of the SK parts of a tile meet in an LDS slot; the wave that arrives last
        // adds them in part order (not arrival order), so the result does not depend on timing
        const int slot = tl & (h.nslot - 1);
        float* rs = red + (size_t)slot * h.sk_cap * h.M * 16;
        if (QB) {
#pragma unroll
          for (int g = 0; g < NG; ++g)
            if (kq + 4 * g < h.M) rs[(part * h.M + kq + 4 * g) * 16 + wr] = part_sum[g];
        } else {
#pragma unroll
          for (int p = 0; p < MP; ++p)
            if (kq == 0 && p < h.M) rs[(part * h.M + p) * 16 + wr] = part_sum[p];
        }
        // release: this wave's partial sums are in LDS before its arrival is counted; acquire: the
        // last arriver reads the other waves' sums only after it has seen all their arrivals
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        int old = 0;
        if (lane == 0) old = atomicAdd(&cnt[slot], 1);
        old = __builtin_amdgcn_readfirstlane(old);                 // lane 0 holds it, and every lane is active here
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        if (old == SK - 1) {                                      // uniform over the wave
          // the partial sums are read four at a time (parts past SK re-read the last one and do
          // not count) and added in part order
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            const int am = kq + 4 * g;                              // quarter kq finishes activation rows kq and 4 + kq
            if (am < h.M) {
              float v = 0.f;
              for (int j0 = 0; j0 < SK; j0 += 4) {
                float pv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) pv[j] = rs[((j0 + j < SK ? j0 + j : SK - 1) * h.M + am) * 16 + wr];
#pragma unroll
                for (int j = 0; j < 4; ++j) v += j0 + j < SK ? pv[j] : 0.f;
              }
              store(am, wr, v);
            }
          }
          if (lane == 0) cnt[slot] = 0;
        }
      }
      }
      p0 = p1; v0 = v1;
      if (v1) v1 = advance(p1);
    };
    while (true) {
      if (!v0) break;
      do_step(LA, LB);
      if (!v0) break;
      do_step(LB, LA);
    }
    // every wave passes the same number of group barriers
    const int ngroups = slabbed ? 1 : ((t_hi - t_lo) + gt - 1) >> gsh;
    for (; bars < ngroups - 1; ++bars) __syncthreads();
    // next trip: the next slab of these tiles, the next group of tiles, the next matrix
    if (SLABS) {
      pa += SP;
      if (pa >= SK) {
        pa = 0;
        g_lo = t_hi;
        if (t_hi >= T_hi) { g_lo = -1; ++mi; }
      }
    } else {
      ++mi;
    }
  }
}

// ------------------------------------------------------------------ long rows, split over the workgroups by columns
// Two to eight activation rows of rows whose digits (M * 3 * N bytes) fill most of LDS or do not
// fit (`down` projections from M = 2 on, 5376 columns from six rows on).  The kernel above has
// every workgroup convert all M x N activations before its first step, and stages a row that
// does not fit slab after slab, with a handful of items per slab for its sixteen wavefronts.
// Here a workgroup owns one column slab (whole parts of the row, the parts of one activation
// row) of a range of tiles of one matrix of the launch: it stages M x (slab) activations once,
// deals the (tile, part) items of its slab to the wavefronts and writes the part sums to a
// caller-provided buffer; a second small kernel adds the parts of every output in part order.
// Same operations in the same order as for one activation row, so a row's result still does not
// depend on M.  Block-per-quarter arrangement only.
struct GsMat {             // one matrix of a column-split launch
  GvMat g;                 // spi, sk: the parts; sp: parts per slab
  int nslab, wps;          // column slabs, workgroups per slab
  int tq, tr;              // ntiles / wps, ntiles % wps
  uint32_t inv_wps;        // b / wps = (b * inv_wps) >> 32 for the matrix's workgroup indices
  int wg0, th0;            // its first workgroup, and its first thread in the reduce launch
  float* part;             // [ntiles][sk][M][16] part sums
};
struct GsHead {
  int n, M, xdt, ydt;
  int xq_cap, delta_cap;   // LDS bytes of digits, floats of delta
  int wg_end[GV_MAX_BATCH];   // workgroups up to and including matrix i (INT_MAX from entry n on)
  int th_end[GV_MAX_BATCH];   // the same for the threads of the reduce launch
};
struct GsArgs {
  GsHead h;
  GsMat mat[GV_MAX_BATCH];
};
static_assert(sizeof(GsArgs) <= 4096 && sizeof(GvBatch) <= 4096, "kernel argument blocks are at most 4 KB");

template <int BITS, int KEEP, int GRP, int MP>
__global__ __launch_bounds__(GV_THREADS) void gemv_split_kernel(GsArgs a) {
  using C = Cfg<BITS, KEEP, GRP, MP>;
  static_assert((MP == 4 || MP == 8) && block_split_capable(BITS, KEEP, GRP), "block-per-quarter configurations only");
  constexpr int NG = MP / 4;                           // groups of four activation rows, one MFMA each per fragment
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  uint2* lut = (uint2*)smem;
  uint8_t* zreg = smem + LUT_BYTES;
  int8_t* xq = (int8_t*)zreg + ZERO_BYTES;
  const GsHead h = a.h;
  float* delta = (float*)(xq + h.xq_cap);
  // the matrix of this workgroup
  int bx = (int)blockIdx.x, mi = 0;
#pragma unroll
  for (int i = 0; i < GV_MAX_BATCH - 1; ++i) mi += bx >= h.wg_end[i] ? 1 : 0;
  const GsMat gs = a.mat[mi];
  bx -= gs.wg0;
  const GvMat& gm = gs.g;
  const DMat& m = gm.m;
  const int M = h.M, N = m.N, NCH = N >> 7, nS = gm.nS, spi = gm.spi, SK = gm.sk;
  if (tid < 256) {
    const uint2 e = make_selectors((uint32_t)tid, C::SEL_KIND);
#pragma unroll
    for (int j = 0; j < LUT_LANES; ++j) lut[tid * LUT_LANES + j] = e;
  } else if (tid < 256 + ZERO_BYTES / 4) {
    ((uint32_t*)zreg)[tid - 256] = 0u;
  } else if (tid < 256 + ZERO_BYTES / 4 + 4 * M) {                  // deltas of the chunks past N
    const int i = tid - 256 - ZERO_BYTES / 4;
    delta[(i >> 2) * (NCH + 4) + NCH + (i & 3)] = 0.f;
  }
  const int wr = lane & 15, kq = lane >> 4;
  const uint32_t l16 = lane & (LUT_LANES - 1);
  const int a_m = wr >> 2, a_dig = wr & 3;             // activation row and digit of this lane's A row
  const uint32_t xq_off = (uint32_t)((uint8_t*)xq - smem), z_off = (uint32_t)(zreg - smem);

  // this workgroup: slab sl, tiles [T_lo, T_hi)
  const int sl = gs.wps == 1 ? bx : (int)__umulhi((uint32_t)bx, gs.inv_wps), wi = bx - sl * gs.wps;
  const int tq = gs.tq, tr = gs.tr;
  const int T_lo = wi * tq + (wi < tr ? wi : tr), T_hi = T_lo + tq + (wi < tr ? 1 : 0);
  const int ntl = T_hi - T_lo;
  if (ntl <= 0) return;                                             // uniform over the workgroup
  const int pa = sl * gm.sp, pn = SK - pa < gm.sp ? SK - pa : gm.sp;        // its parts
  const int S0 = pa * spi, S1 = (pa + pn) * spi < nS ? (pa + pn) * spi : nS;
  const int col0 = S0 * 512, Ns = N - col0 < (S1 - S0) * 512 ? N - col0 : (S1 - S0) * 512, ch0 = col0 >> 7;

  const uint8_t* const m_data = m.data;
  const uint16_t* const m_scale = m.scale;
  const uint8_t* const m_zero = m.zero;
  const int m_K = m.K, m_G = m.G, ush = gm.ush, csh = gm.csh;
  const uint32_t tile_a = gm.tile_a, lane_mul = gm.lane_mul, sz_mul = gm.sz_mul, code_u0 = m.code_off >> 4;
  const int last_S = nS - 1, last_tile = T_hi - 1;

  // loads of one (tile, macro-step) position: block kq of the chunks 4S .. 4S+3 of row wr
  auto issue = [&](int tile, int S, Loads<C>& L) {
    tile = tile < last_tile ? tile : last_tile;
    S = S < last_S ? S : last_S;
    const int S4 = 4 * S;
    const int rlim = m_K - 1 - tile * 16;                           // rows past K repeat row K - 1
    const uint32_t wrc = (uint32_t)(wr < rlim ? wr : rlim);
    const uint32_t lane_off = __umul24(wrc, lane_mul);
    const int klim = NCH - 1 - S4;                                  // chunks past N repeat chunk NCH - 1
    const uint32_t chl = (uint32_t)(kq < klim ? kq : klim);
    const uint32_t so_t = (uint32_t)tile * tile_a;
    const uint32_t so_g = (uint32_t)tile * (uint32_t)(16 * m_G);
    constexpr uint32_t BB = C::CB / 8;
    const uint32_t voff_m = lane_off + (uint32_t)kq * 4u;
    const uint32_t voff_c = lane_off + ((((uint32_t)kq * BB) >> 4) << ush) + (((uint32_t)kq * BB) & 15u);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      int chc = S4 + c;
      chc = chc < NCH ? chc : NCH - 1;
      if (!C::DENSE) L.mk[c] = *(const uint32_t*)(m_data + (so_t + ((uint32_t)chc << ush) + voff_m));
      const uint8_t* cp = m_data + (so_t + ((code_u0 + (uint32_t)chc * (C::CHB / 128)) << ush) + voff_c);
      if (C::CB == 32) {
        L.raw[c] = *(const uint32_t*)cp;
      } else if (C::CB == 64) {
        const uint2 v = *(const uint2*)cp;
        L.raw[2 * c] = v.x; L.raw[2 * c + 1] = v.y;
      } else {
        const uint4 v = *(const uint4*)cp;
        L.raw[4 * c] = v.x; L.raw[4 * c + 1] = v.y; L.raw[4 * c + 2] = v.z; L.raw[4 * c + 3] = v.w;
      }
    }
    const uint32_t gv = so_g + ((uint32_t)S4 << csh) + __umul24(wrc, sz_mul) + (chl << csh);
    L.zraw = (uint32_t)m_zero[gv] | ((uint32_t)m_scale[gv] << 8);
  };

  // this wave's (tile, part, macro-step) positions: items wave, wave + 16, ... of the slab
  struct Pos { int tl, part, S; };
  const bool whole = pn == gm.sp;                                  // (a shorter last slab divides in software)
  const int dq_t = whole ? gm.dq_t : GV_WAVES / pn, dq_p = whole ? gm.dq_p : GV_WAVES % pn;
  const int w_t = whole ? (int)(((uint32_t)wave * gm.inv_sp) >> 16) : wave / pn, w_p = wave - w_t * pn;
  auto advance = [&](Pos& p) -> bool {                             // false past the last position
    const int s_end = (p.part * spi + spi < nS) ? p.part * spi + spi : nS;
    if (p.S + 1 < s_end) { ++p.S; return true; }
    p.tl += dq_t; p.part += dq_p;
    if (p.part >= pa + pn) { p.part -= pn; ++p.tl; }
    p.S = p.part * spi;
    return p.tl < ntl;
  };
  Pos p0{w_t, pa + w_p, (pa + w_p) * spi};
  bool v0 = p0.tl < ntl;
  Pos p1 = p0; bool v1 = v0 && advance(p1);

  // ---- stage the slab's digits (the activation loads go out before the first weight loads)
  constexpr int XORD = !C::DENSE ? 0 : (BITS == 2 ? 2 : 1);
  const int n16 = Ns >> 4, xitems = M * n16;                        // a multiple of 8
  XLoad xl;
  if (tid < xitems) stage_load(gm.x, gm.ldx, m.cs, N, col0, n16, tid, false, gm.par, xl);
  Loads<C> LA, LB;
  issue(T_lo + p0.tl, p0.S, LA);
  if (tid < xitems) stage_convert<XORD>(xl, m.cs != nullptr, h.xdt, N, ch0, n16, tid, false, xq, delta, X_PAD);
  for (int xit = tid + GV_THREADS; xit < xitems; xit += GV_THREADS) {
    stage_load(gm.x, gm.ldx, m.cs, N, col0, n16, xit, false, gm.par, xl);
    stage_convert<XORD>(xl, m.cs != nullptr, h.xdt, N, ch0, n16, xit, false, xq, delta, X_PAD);
  }
  __syncthreads();

  float ysum[MP];
  auto do_step = [&](Loads<C>& cur, Loads<C>& tgt) {               // decode `cur`, load the next step into `tgt`
    const int tl = p0.tl, part = p0.part, S = p0.S;
    const int tile = T_lo + tl;
    const int s_end = (part * spi + spi < nS) ? part * spi + spi : nS;
    if (S == part * spi) {
#pragma unroll
      for (int p = 0; p < MP; ++p) ysum[p] = 0.f;
    }
    issue(T_lo + p1.tl, p1.S, tgt);
    uint32_t zs[4];                                                 // zero | scale << 8 of the groups 4S .. 4S+3
#pragma unroll
    for (int c = 0; c < 4; ++c) zs[c] = (uint32_t)__shfl((int)cur.zraw, wr + 16 * c, 64);
    bool a_on[NG];
    uint32_t a_base[NG];
    int dm[NG];                                                     // the activation rows this quarter sums
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      a_on[g] = a_dig < NDIG && a_m + 4 * g < M;
      a_base[g] = xq_off + (uint32_t)(((a_m + 4 * g) * NDIG + a_dig) * (Ns + X_PAD) + kq * 32);
      dm[g] = kq + 4 * g < M ? kq + 4 * g : 0;
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int chunk = 4 * S + c;
      uint32_t aaddr[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) aaddr[g] = (a_on[g] && chunk < NCH) ? a_base[g] + (uint32_t)(chunk - ch0) * 128u : z_off;
      uint32_t rkc[4];
      uint2 selc[4];
      fetch_selectors<C>(cur.mk[c], lut, l16, rkc, selc);
      uint32_t st[C::NW];
#pragma unroll
      for (int k = 0; k < C::NW; ++k) st[k] = cur.raw[c * C::NW + k];
      const uint32_t z = zs[c] & 0xFFu;
      const uint32_t nz = 0x80808080u - z * 0x01010101u;
      v4i acc[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) acc[g] = (v4i){0, 0, 0, 0};
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint32_t bfrag[4];
        decode_half<C, BITS>(st, rkc, selc, nz, half, bfrag);
        const v4i bv = (v4i){(int)bfrag[0], (int)bfrag[1], (int)bfrag[2], (int)bfrag[3]};
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const v4i av = *(const v4i*)(smem + aaddr[g] + 16 * half);
          acc[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[g], 0, 0, 0);
          asm("s_nop 1" : "+v"(acc[g]));                            // see the main kernel
        }
      }
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const float dl = delta[dm[g] * (NCH + 4) + chunk];          // 0 past the last chunk
        const float f = fmaf((float)(acc[g][0] * 256 + acc[g][1]), 256.f, (float)acc[g][2]);
        ysum[4 * g + c] = fmaf(f, h2f((uint16_t)(zs[c] >> 8)) * dl, ysum[4 * g + c]);
      }
    }
    if (S + 1 == s_end) {
      // the part is done: lane quarter kq holds activation row 4g + kq of weight row wr
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const float ps = (ysum[4 * g] + ysum[4 * g + 1]) + (ysum[4 * g + 2] + ysum[4 * g + 3]);
        if (kq + 4 * g < M) gs.part[((size_t)(tile * SK + part) * M + kq + 4 * g) * 16 + wr] = ps;
      }
    }
    p0 = p1; v0 = v1;
    if (v1) v1 = advance(p1);
  };
  while (true) {
    if (!v0) break;
    do_step(LA, LB);
    if (!v0) break;
    do_step(LB, LA);
  }
}

// the parts of every output, added in part order; bias; conversion
constexpr int GS_RED_THREADS = 256;
static inline size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }
static inline size_t split_part_bytes(int ntiles, int sk, int Mk) { return (size_t)ntiles * sk * Mk * 16 * 4; }   // [tiles][parts][M][16] floats
__global__ __launch_bounds__(GS_RED_THREADS) void gemv_split_reduce_kernel(GsArgs a) {
  const GsHead& h = a.h;
  int idx = (int)blockIdx.x * GS_RED_THREADS + (int)threadIdx.x, mi = 0;
#pragma unroll
  for (int i = 0; i < GV_MAX_BATCH - 1; ++i) mi += idx >= h.th_end[i] ? 1 : 0;     // (uniform over the workgroup)
  const GsMat& gs = a.mat[mi];
  idx -= gs.th0;
  const GvMat& gm = gs.g;
  const int M = h.M, SK = gm.sk;
  const int wr = idx & 15, t = idx >> 4, tile = t / M, am = t - tile * M;
  if (tile >= gm.ntiles) return;
  const int k = tile * 16 + wr;
  if (k >= gm.m.K) return;
  int om = am;
  if (gm.par) {                                                     // the sum scaled for the other parity is dropped
    if ((om ^ k) & 1) return;
    om >>= 1;
  }
  float pv[16];                                                     // all loads first (at most 16 parts), then the sum in part order
#pragma unroll
  for (int j = 0; j < 16; ++j) pv[j] = gs.part[((size_t)(tile * SK + (j < SK ? j : SK - 1)) * M + am) * 16 + wr];
  float v = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) v += j < SK ? pv[j] : 0.f;
  if (gm.bias) v += (h.ydt == CBK_F32) ? ((const float*)gm.bias)[k]
                  : (h.ydt == CBK_F16) ? h2f(((const uint16_t*)gm.bias)[k]) : bf2f(((const uint16_t*)gm.bias)[k]);
  const size_t o = (size_t)om * gm.ldy + k;
  if (h.ydt == CBK_F32) ((float*)gm.y)[o] = v;
  else if (h.ydt == CBK_F16) ((uint16_t*)gm.y)[o] = f2h(v);
  else ((uint16_t*)gm.y)[o] = f2bf(v);
}

// ------------------------------------------------------------------ survivor-stream rows
// SPARSE4 / SPARSE4X / SPARSE4E at one to eight activation rows per pass.  Rows of different lengths do not
// tile, so there is no matrix-core kernel for them; but the float row kernel spends about fourteen
// vector instructions per column (pruned ones included) and is bound by that.  This kernel keeps
// the arithmetic of the kernel above (activation digits in LDS, byte-permute expansion of the
// bitmap into signed bytes q - zero, exact int32 sums per digit, one float FMA per 32-column block
// with scale * delta) and forms the sums with v_dot4_i32_i8: about seven instructions per column.
// One wavefront per weight row, one lane per 32-column block; a persistent workgroup of sixteen
// wavefronts per CU stages the digits once and then walks rows.
// Reference semantics: cbk::gemv_sparse4 (src/cobaltkernel/csrc/cobalt_gemv.cuh:216-301).
constexpr int ST_WAVES = 16;
constexpr int ST_THREADS = ST_WAVES * 64;
constexpr int ST_LUT_LANES = 4;
constexpr int ST_LUT_BYTES = 256 * ST_LUT_LANES * 8;
constexpr int ST_X_BUDGET = 96 * 1024;        // digits of all activation rows of a pass
constexpr int ST_MAX_M = 8;                   // activation rows per pass

// What a lane fetches for one (row, 32-column block) item, in two dependent steps: the group's mask
// words and code offset, then (at an address made from those) the block's codes and the group's
// scale and zero point.
struct StMask { uint4 gmk; uint32_t goffv; };
struct StCodes { uint32_t e[5]; uint32_t mw, sh, sraw, z; };

template <int M>
__global__ __launch_bounds__(ST_THREADS) void gemv_stream_kernel(DMat m, const uint16_t* x, int64_t ldx, int xdt,
                                                                 void* y, int ydt, int64_t ldy, const void* bias) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint2* lut = (uint2*)smem;
  const int N = m.N, NCH = N >> 7, NB = N >> 5;
  int8_t* xq = (int8_t*)(smem + ST_LUT_BYTES);
  float* delta = (float*)(xq + (size_t)M * NDIG * N);
  uint32_t* goffs = (uint32_t*)(delta + M * (NCH + 4));          // [ST_WAVES][G], SPARSE4 only
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool has_goff = m.layout != CBK_SPARSE4;
  const int hdr = ((N >> 3) + (has_goff ? ((m.G * 2 + 15) & ~15) : 0) + 15) & ~15;
  uint32_t* lgoff = goffs + wave * m.G;
  const uint32_t l4 = lane & (ST_LUT_LANES - 1);
  // this wavefront's rows k0, k0 + ks, ...; its items are (row, pass over the row's blocks), in order
  // (a wavefront without rows goes through the first loads on the last row and leaves after the barrier)
  const int kw = (int)blockIdx.x * ST_WAVES + wave, ks = (int)gridDim.x * ST_WAVES;
  const int k0 = kw < m.K ? kw : m.K - 1;
  const int nrows = kw < m.K ? (m.K - k0 + ks - 1) / ks : 0;
  const int nt = (NB + 63) >> 6, nitems = nrows * nt;
  const uint8_t* const m_data = m.data;
  const uint32_t* const m_row_off = m.row_off;

  // Items run through a three-deep pipeline: while item q is multiplied, the codes of item q + 1
  // and the mask words of item q + 2 are on their way.  Positions past the end repeat the last item.
  struct Pos { int k, it; uint32_t ro; };
  auto next_pos = [&](Pos& p) {
    if (p.it + 1 < nt) { ++p.it; return; }
    if (p.k + ks < m.K) { p.k += ks; p.it = 0; p.ro = m_row_off[p.k]; }
  };
  auto block_of = [&](const Pos& p) { const int t = lane + 64 * p.it; return t < NB ? t : NB - 1; };
  auto issue_mask = [&](const Pos& p, StMask& a) {
    const int g = block_of(p) >> 2;
    const uint8_t* row = m_data + p.ro;
    a.gmk = ((const uint4*)row)[g];                               // the four mask words of the group
    a.goffv = has_goff ? (uint32_t)((const uint16_t*)(row + (N >> 3)))[g] : 0u;
  };
  auto issue_codes = [&](const Pos& p, const StMask& a, StCodes& c) {
    const int t = block_of(p), g = t >> 2, j = t & 3;
    const uint8_t* row = m_data + p.ro;
    if (!has_goff && p.it == 0) {
      // SPARSE4: the byte offset of every group's codes is a prefix sum of the groups' byte counts
      const uint32_t* bm = (const uint32_t*)row;
      uint32_t carry = 0;
      for (int g0 = 0; g0 < m.G; g0 += 64) {
        const int gg = g0 + lane;
        uint32_t nb = 0;                                          // bytes of group gg: an even number of nibbles
        if (gg < m.G) {
          const uint4 v = ((const uint4*)bm)[gg];
          nb = (uint32_t)(__popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w) + 1) >> 1;
        }
        uint32_t incl = nb;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const uint32_t v = (uint32_t)__shfl_up((int)incl, o, 64);
          incl += lane >= o ? v : 0u;
        }
        if (gg < m.G) lgoff[gg] = carry + incl - nb;
        carry += (uint32_t)__shfl((int)incl, 63, 64);
      }
      __builtin_amdgcn_wave_barrier();
    }
    c.mw = j == 0 ? a.gmk.x : j == 1 ? a.gmk.y : j == 2 ? a.gmk.z : a.gmk.w;
    const uint32_t pre = (j > 0 ? __popc(a.gmk.x) : 0) + (j > 1 ? __popc(a.gmk.y) : 0) + (j > 2 ? __popc(a.gmk.z) : 0);
    const uint8_t* cp = row + hdr + (has_goff ? a.goffv : lgoff[g]) + (pre >> 1);
    const uintptr_t ca = (uintptr_t)cp & ~(uintptr_t)3;
    c.sh = (uint32_t)(((uintptr_t)cp & 3) * 8 + (pre & 1) * 4);   // < 32
#pragma unroll
    for (int i = 0; i < 5; ++i) c.e[i] = ((const uint32_t*)ca)[i];               // 16 bytes + skew; rows end in a readable tail
    c.sraw = m.scale[(size_t)p.k * m.G + g];
    c.z = m.zero[(size_t)p.k * m.G + g];
  };

  float ysum[M];
#pragma unroll
  for (int i = 0; i < M; ++i) ysum[i] = 0.f;
  auto compute = [&](const Pos& p, const StCodes& c) {
    const int traw = lane + 64 * p.it;
    const bool valid = traw < NB;
    const int t = valid ? traw : NB - 1, g = t >> 2;
    uint32_t w[4];                                                // the block's codes (at most 32 nibbles) from bit 0 on
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = __builtin_amdgcn_alignbit(c.e[i + 1], c.e[i], c.sh);
    const uint32_t mw = c.mw;
    const uint32_t nz = 0x80808080u - c.z * 0x01010101u;
    int acc[M][NDIG];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int d = 0; d < NDIG; ++d) acc[i][d] = 0;
    // The lanes take the four mask bytes of their blocks in different orders (byte jb ^ rot in
    // turn jb): a lane's digits are 32 bytes from its neighbour's, and with every lane on the same
    // byte of its block the 8-byte reads of 32 lanes would fall on eight of the 64 LDS banks.
    const uint32_t rot = ((uint32_t)lane >> 3) & 3u;
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const uint32_t jl = (uint32_t)jb ^ rot;
      const uint32_t mb = (mw >> (8u * jl)) & 0xFFu;
      const uint32_t r = (uint32_t)__popc(mw & ~(0xFFFFFFFFu << (8u * jl)));                 // survivors before this byte
      // 32 bits of the stream from nibble r on (r <= 24, and a shift of 0 at r = 24): dwords r / 8 and
      // r / 8 + 1, picked with two levels of bitwise selects under the sign-extended bits 4 and 3 of r
      const uint32_t m64 = (uint32_t)__builtin_amdgcn_sbfe((int)r, 4, 1), m32 = (uint32_t)__builtin_amdgcn_sbfe((int)r, 3, 1);
      const uint32_t x0 = mask_select(m64, w[0], w[2]), x1 = mask_select(m64, w[1], w[3]), x2 = w[2] & ~m64;
      const uint32_t lo = mask_select(m32, x0, x1), hi = mask_select(m32, x1, x2);
      const uint32_t win = __builtin_amdgcn_alignbit(hi, lo, (r & 7u) * 4u);
      const uint32_t p0 = bias_pool(win & 0x0F0F0F0Fu, nz), p1 = bias_pool((win >> 4) & 0x0F0F0F0Fu, nz);
      const uint2 sel = lut[mb * ST_LUT_LANES + l4];
      const int b0 = (int)perm(p1, p0, sel.x), b1 = (int)perm(p1, p0, sel.y);   // q - zero of columns 0-3, 4-7; pruned: 0
      const int c0 = t * 32 + 8 * (int)jl;
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int d = 0; d < NDIG; ++d) {
          const uint2 a = *(const uint2*)(xq + (size_t)(i * NDIG + d) * N + c0);
          acc[i][d] = __builtin_amdgcn_sdot4(b0, (int)a.x, acc[i][d], false);
          acc[i][d] = __builtin_amdgcn_sdot4(b1, (int)a.y, acc[i][d], false);
        }
    }
    const float s = valid ? h2f((uint16_t)c.sraw) : 0.f;
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const float f = fmaf((float)(acc[i][0] * 256 + acc[i][1]), 256.f, (float)acc[i][2]);
      ysum[i] = fmaf(f, s * delta[i * (NCH + 4) + g], ysum[i]);
    }
    if (p.it + 1 == nt) {                                         // the row is complete
      const int k = p.k;
#pragma unroll
      for (int i = 0; i < M; ++i) {
        const float v0 = ysum[i];
        ysum[i] = 0.f;
        float v = wave_sum_dpp(v0);
        if (lane == 0) {
          if (bias) v += (ydt == CBK_F32) ? ((const float*)bias)[k]
                       : (ydt == CBK_F16) ? h2f(((const uint16_t*)bias)[k]) : bf2f(((const uint16_t*)bias)[k]);
          if (ydt == CBK_F32) ((float*)y)[(size_t)i * ldy + k] = v;
          else if (ydt == CBK_F16) ((uint16_t*)y)[(size_t)i * ldy + k] = f2h(v);
          else ((uint16_t*)y)[(size_t)i * ldy + k] = f2bf(v);
        }
      }
    }
  };

  Pos pc{k0, 0, m_row_off[k0]};                                   // item being multiplied
  Pos pb = pc;                                                    // item whose codes are being fetched
  StMask am;
  StCodes ca, cb;                                                 // swap roles by name (a copy would wait for the loads)
  issue_mask(pc, am);
  issue_codes(pc, am, ca);
  next_pos(pb);
  Pos pa = pb;                                                    // item whose mask words are being fetched
  issue_mask(pb, am);
  // Selector table and activation digits, while the first rows' bytes are on their way (three
  // dependent loads: row offset, mask words, codes).
  if (tid < 256) {
    const uint2 e = make_selectors((uint32_t)tid, 0);
#pragma unroll
    for (int j = 0; j < ST_LUT_LANES; ++j) lut[tid * ST_LUT_LANES + j] = e;
  }
  const int n16 = N >> 4, xitems = M * n16;                      // a multiple of 8
  for (int it = tid; it < xitems; it += ST_THREADS) {
    XLoad xl;
    stage_load(x, ldx, m.cs, N, 0, n16, it, M == 1, 0, xl);
    stage_convert<0>(xl, m.cs != nullptr, xdt, N, 0, n16, it, M == 1, xq, delta);
  }
  __syncthreads();
  if (kw >= m.K) return;
  for (int q = 0; q < nitems; q += 2) {
    issue_codes(pb, am, cb);
    next_pos(pa);
    issue_mask(pa, am);
    compute(pc, ca);
    pc = pb; pb = pa;
    if (q + 1 >= nitems) break;
    issue_codes(pb, am, ca);
    next_pos(pa);
    issue_mask(pa, am);
    compute(pc, cb);
    pc = pb; pb = pa;
  }
}

template <int M>
static int launch_stream_m(const DMat& m, const void* x, int64_t ldx, int xdt, void* y, int ydt, int64_t ldy,
                           const void* bias, hipStream_t st) {
  auto kern = gemv_stream_kernel<M>;
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  const size_t lds = (size_t)ST_LUT_BYTES + (size_t)M * NDIG * m.N + (size_t)M * (m.N / 128 + 4) * 4 +
                     (m.layout == CBK_SPARSE4 ? (size_t)ST_WAVES * m.G * 4 : 0);
  if (lds > 160 * 1024) return CBK_ERR_UNSUPPORTED;
  int blocks = (m.K + ST_WAVES - 1) / ST_WAVES;
  blocks = blocks < 256 ? blocks : 256;                           // one persistent workgroup per CU
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(ST_THREADS), lds, st, m, (const uint16_t*)x, ldx, xdt, y, ydt, ldy, bias);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

// ------------------------------------------------------------------ survivor-stream rows on the matrix cores
// SPARSE4X / SPARSE4E (a code offset per group in the row) in 16-row tiles on the 16x16x64 int8
// MFMA, block-per-quarter arrangement: lane (weight row wr, quarter kq) decodes block kq of each
// of the four groups of a 512-column step, one MFMA covers 64 columns of one group for up to four
// activation rows, a second one the rows 4..7.  The rows of a tile have different lengths, so
// every lane finds its codes itself: the group's mask words and code offset are loaded a step
// ahead of the codes, whose address they give (survivors in the group's earlier blocks).  A lane
// loads the mask words and the offset of one group (group 4S + kq), forms the nibble address of
// each of its four blocks, and the four lanes of a weight row exchange what they hold with a
// 4 x 4 transpose over the lane quarters (four row-swap instructions per register set).  Against
// the row kernel above: the dot products and the digit reads of every activation row are gone
// (about half the instructions at one activation row), and the time hardly grows with M.
//
// Work split: a workgroup takes a range of tiles; a tile's row is cut into SK parts of spi steps,
// wavefront w of a round works on part w % SK of the round's tile w / SK; the part sums meet in
// LDS and are added in part order: by the wavefront that finishes a tile's round last, or (BAR,
// used for one activation row, where it measured faster) by all threads behind a barrier.  SK
// and spi depend on the matrix shape only, and every activation row goes through the same
// operations in the same order whatever M is.  SPLIT: for activation rows that do not fit in LDS
// as whole rows a workgroup takes one column slab (some of the SK parts) of a range of tiles and
// writes its part sums to the caller's workspace; gemv_split_reduce_kernel adds them, in the
// same order.
// Reference semantics: cbk::gemv_sparse4 (src/cobaltkernel/csrc/cobalt_gemv.cuh:216-301).
struct SmArgs {
  DMat m;
  const uint16_t* x;
  int64_t ldx;
  void* y;
  int64_t ldy;
  const void* bias;
  int M, xdt, ydt;         // M: activation rows as the kernel counts them
  int par;                 // 1: two col_scale vectors by row parity (a fused gate/up matrix): kernel row v is row v / 2 of
                           // x scaled by vector v % 2, and weight row k keeps the rows v = k (mod 2)
  int ntiles, tq, tr;      // tiles per workgroup: tq, one more for the first tr workgroups
  int nS, spi, sk;         // steps per row, steps per part, parts
  uint32_t inv_sk;         // w / sk = (w * inv_sk) >> 16 for w < 16
  int hdr;                 // bytes of a row before its codes
  // column-split launches: a workgroup owns pps consecutive parts (one column slab) of a range of
  // tiles, wps workgroups per slab (tq, tr: tiles over the workgroups of a slab), and writes the
  // part sums to part[tile][sk][M][16]
  int pps, wps;
  float* part;
};
struct SmMask { uint4 mk; uint32_t go; };                           // mask words and code offset of group 4S + kq
struct SmCodes { uint32_t e[4][5]; uint32_t mw[4], sh[4]; uint32_t zs; };   // codes (16 bytes + skew), mask word, bit skew per group

template <int NG, bool BAR, bool SPLIT>
__global__ __launch_bounds__(GV_THREADS) void gemv_stream_mfma_kernel(SmArgs a) {
  static_assert(!(BAR && SPLIT), "a column-split launch adds nothing itself");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const DMat& m = a.m;
  const int M = a.M, N = m.N, NCH = N >> 7;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int spi = a.spi, nS = a.nS;
  // the workgroup's parts [p_lo, p_lo + SK) of the a.sk parts of a row, its columns and tiles
  const int sl = SPLIT ? (int)blockIdx.x / a.wps : 0;
  const int bx = SPLIT ? (int)blockIdx.x - sl * a.wps : (int)blockIdx.x;
  const int p_lo = SPLIT ? sl * a.pps : 0;
  const int SK = SPLIT ? (a.sk - p_lo < a.pps ? a.sk - p_lo : a.pps) : a.sk;
  const int col0 = p_lo * spi * 512;
  const int cols = SPLIT ? (N - col0 < SK * spi * 512 ? N - col0 : SK * spi * 512) : N;
  const int ch0 = col0 >> 7, Ns = cols + X_PAD;
  uint2* lut = (uint2*)smem;
  uint8_t* zreg = smem + LUT_BYTES;
  int* arrived = (int*)(zreg + ZERO_BYTES);                       // [2][16] part sums written, by round parity and tile of the round
  int* summed = arrived + 2 * GV_WAVES;                           // [16] rounds whose part sums have been added
  int8_t* xq = (int8_t*)zreg + ZERO_BYTES + CNT_BYTES;
  float* delta = (float*)(xq + (size_t)M * NDIG * (SPLIT ? a.pps * spi * 512 + X_PAD : Ns));
  float* red = delta + M * (NCH + 4);                             // [2][M][16 wavefronts][16 rows], by round parity
  const int wr = lane & 15, kq = lane >> 4;
  const uint32_t l16 = lane & (LUT_LANES - 1);
  const int T_lo = bx * a.tq + (bx < a.tr ? bx : a.tr), T_hi = T_lo + a.tq + (bx < a.tr ? 1 : 0);
  const int TPR = GV_WAVES / SK;                                  // tiles per round (scalar, once)
  const int R = (T_hi - T_lo + TPR - 1) / TPR;                    // rounds
  const int tir = SPLIT ? wave / SK : (int)(((uint32_t)wave * a.inv_sk) >> 16);
  const int part = p_lo + wave - tir * SK;
  const bool idle = tir >= TPR;                                   // wavefronts past the last whole tile of a round
  const int s0 = part * spi, s1 = s0 + spi < nS ? s0 + spi : nS;  // this wavefront's steps (never empty: host)
  const uint8_t* const m_data = m.data;
  const uint32_t* const m_row_off = m.row_off;
  const int m_K = m.K, m_G = m.G;
  const uint32_t hdr = (uint32_t)a.hdr, go_off = (uint32_t)(N >> 3);

  auto tile_of = [&](int round) { const int t = T_lo + round * TPR + (idle ? 0 : tir); return t < T_hi ? t : T_hi - 1; };
  auto row_of = [&](int tile) { const int k = tile * 16 + wr; return k < m_K ? k : m_K - 1; };

  // Positions (round, step) of this wavefront, in order; past the last one it repeats.  The row
  // offsets of a round's tile are fetched a round ahead.
  struct Pos { int round, S; uint32_t ro; };
  uint32_t ro_next = m_row_off[row_of(tile_of(1 < R ? 1 : 0))];
  auto advance = [&](Pos& p) {
    if (p.S + 1 < s1) { ++p.S; return; }
    if (p.round + 1 >= R) return;
    ++p.round; p.S = s0; p.ro = ro_next;
    ro_next = m_row_off[row_of(tile_of(p.round + 1 < R ? p.round + 1 : p.round))];
  };
  auto issue_mask = [&](const Pos& p, SmMask& k) {
    const uint8_t* row = m_data + p.ro;
    int g = 4 * p.S + kq;
    g = g < m_G ? g : m_G - 1;                                      // groups past the row repeat the last one
    k.mk = ((const uint4*)row)[g];
    k.go = (uint32_t)((const uint16_t*)(row + go_off))[g];
  };
  // r0..r3 hold, in lane quarter q, the values (q, 0..3); afterwards register i holds (i, q):
  // the upper two quarters of r0 / r1 change places with the lower two of r2 / r3, then the odd
  // quarters of r0 / r2 with the even ones of r1 / r3.  (Inline assembly as in quarter_sum.)
  auto transpose4 = [&](uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(r0), "+v"(r2));
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(r1), "+v"(r3));
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(r0), "+v"(r1));
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(r2), "+v"(r3));
  };
  auto issue_codes = [&](const Pos& p, const SmMask& k, SmCodes& c) {
    const uint32_t cbase = p.ro + hdr;                              // the row's codes (16-byte aligned)
    // nibble address, in the row's codes, of the four blocks of this lane's group
    const uint32_t n0 = 2u * k.go;
    const uint32_t n1 = n0 + (uint32_t)__popc(k.mk.x), n2 = n1 + (uint32_t)__popc(k.mk.y), n3 = n2 + (uint32_t)__popc(k.mk.z);
    uint32_t na[4] = {n0, n1, n2, n3};
    c.mw[0] = k.mk.x; c.mw[1] = k.mk.y; c.mw[2] = k.mk.z; c.mw[3] = k.mk.w;
    transpose4(c.mw[0], c.mw[1], c.mw[2], c.mw[3]);                 // now of block kq of the groups 4S .. 4S+3
    transpose4(na[0], na[1], na[2], na[3]);
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) {
      c.sh[ci] = na[ci] << 2;                                       // (used modulo 32: the nibble inside the dword)
      const uint32_t* cp = (const uint32_t*)(m_data + (cbase + ((na[ci] >> 1) & ~3u)));
#pragma unroll
      for (int i = 0; i < 4; ++i) c.e[ci][i] = cp[i];               // rows end in a readable tail
      // A fifth dword only where the block's survivors reach into it (more than 25 of 32 kept, or
      // fewer behind a skew): as a second load of the cache line the first one has just
      // requested it would wait in the cache for that line, and every wavefront behind it.
      c.e[ci][4] = 0u;
      if ((na[ci] & 7u) + (uint32_t)__popc(c.mw[ci]) > 32u) c.e[ci][4] = cp[4];
    }
    int g = 4 * p.S + kq;
    g = g < m_G ? g : m_G - 1;
    const size_t gi = (size_t)row_of(tile_of(p.round)) * m_G + g;
    c.zs = (uint32_t)m.zero[gi] | ((uint32_t)m.scale[gi] << 8);    // of group 4S + kq; the other quarters fetch it from this lane
  };

  // role of this lane's row in the A operand: activation row a_m (+ 4 per row group), digit a_dig
  // (digit 3 is an all-zero row); in the result, lane quarter kq holds the three digit sums of
  // activation row kq (+ 4 per row group) for weight row wr
  const int a_m = wr >> 2, a_dig = wr & 3;
  const uint32_t xq_off = (uint32_t)((uint8_t*)xq - smem), z_off = (uint32_t)(zreg - smem);
  bool a_on[NG];
  uint32_t a_base[NG];
  int dm[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    a_on[g] = a_dig < NDIG && a_m + 4 * g < M;
    a_base[g] = xq_off + (uint32_t)(((a_m + 4 * g) * NDIG + a_dig) * Ns + kq * 32);
    dm[g] = kq + 4 * g < M ? kq + 4 * g : 0;
  }

  float ysum[4 * NG];
#pragma unroll
  for (int i = 0; i < 4 * NG; ++i) ysum[i] = 0.f;

  auto emit = [&](int am, int k, float v) {
    if (a.par) {                                                    // the sum scaled for the other parity is dropped
      if ((am ^ k) & 1) return;
      am >>= 1;
    }
    const size_t oi = (size_t)am * a.ldy + k;
    if (a.ydt == CBK_F32) ((float*)a.y)[oi] = v;
    else if (a.ydt == CBK_F16) ((uint16_t*)a.y)[oi] = f2h(v);
    else ((uint16_t*)a.y)[oi] = f2bf(v);
  };
  // (Two separate paths on purpose.  With the bias added behind a common join the wait for its
  // load stood there for calls without a bias too, and a wait for a load issued last is a wait
  // for every load in flight, the next step's codes and mask words included: once per round,
  // in the wavefront that was last already.)
  auto store = [&](int am, int tile, float v) {
    const int k = tile * 16 + wr;
    if (k >= m_K) return;
    if (a.bias) {
      const float b = (a.ydt == CBK_F32) ? ((const float*)a.bias)[k]
                    : (a.ydt == CBK_F16) ? h2f(((const uint16_t*)a.bias)[k]) : bf2f(((const uint16_t*)a.bias)[k]);
      emit(am, k, v + b);
    } else {
      emit(am, k, v);
    }
  };

  // BAR: the part sums of a round, added in part order by all threads after the round's barrier
  auto finish_round = [&](int round) {
    const float* rb = red + (size_t)(round & 1) * M * 256;
    for (int o = tid; o < M * 256; o += GV_THREADS) {
      const int r = o & 15, t = (o >> 4) & 15, am = o >> 8;
      const int tile = T_lo + round * TPR + t;
      const int k = tile * 16 + r;
      if (t >= TPR || tile >= T_hi || k >= m_K) continue;
      float pv[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) pv[j] = rb[(am * 16 + t * SK + (j < SK ? j : SK - 1)) * 16 + r];
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) v += j < SK ? pv[j] : 0.f;
      if (a.bias) v += (a.ydt == CBK_F32) ? ((const float*)a.bias)[k]
                     : (a.ydt == CBK_F16) ? h2f(((const uint16_t*)a.bias)[k]) : bf2f(((const uint16_t*)a.bias)[k]);
      emit(am, k, v);
    }
  };

  auto compute = [&](const Pos& p, const SmCodes& c) {
    const int S = p.S;
    uint32_t zs[4];
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) zs[ci] = (uint32_t)__shfl((int)c.zs, wr + 16 * ci, 64);
    // (uniform over the wavefront: in the last round a wavefront may be left without a tile; it
    // has loaded the last tile again and multiplies nothing)
    const bool live = T_lo + p.round * TPR + tir < T_hi;
    if (live)
#pragma unroll
    for (int ci = 0; ci < 4; ++ci) {
      const int chunk = 4 * S + ci;
      uint32_t aaddr[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) aaddr[g] = (a_on[g] && chunk < NCH) ? a_base[g] + (uint32_t)(chunk - ch0) * 128u : z_off;
      uint32_t w[4];                                                // the block's codes from bit 0 on
#pragma unroll
      for (int i = 0; i < 4; ++i) w[i] = __builtin_amdgcn_alignbit(c.e[ci][i + 1], c.e[ci][i], c.sh[ci]);
      const uint32_t mw = c.mw[ci];
      uint32_t mb[4], rk[4];
      mb[0] = mw & 0xFFu; mb[1] = __builtin_amdgcn_ubfe(mw, 8, 8); mb[2] = __builtin_amdgcn_ubfe(mw, 16, 8); mb[3] = mw >> 24;
      rk[1] = (uint32_t)__popc(mb[0]);                              // <= 8
      rk[2] = rk[1] + (uint32_t)__popc(mb[1]);                      // <= 16
      rk[3] = rk[2] + (uint32_t)__popc(mb[2]);                      // <= 24
      uint2 sel[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) sel[j] = lut[mb[j] * LUT_LANES + l16];
      // 32 bits of the stream from nibble rk[j] on
      uint32_t win[4];
      win[0] = w[0];
      win[1] = (uint32_t)((((uint64_t)w[1] << 32) | w[0]) >> (4u * rk[1]));
      {
        // the 64 bits from nibble rk[2] (<= 16) on: dwords r / 8 .. r / 8 + 2 of w[0..3], then the
        // window of the fourth mask byte is those 64 bits shifted by the third byte's survivors
        const uint32_t r = rk[2];
        const uint32_t m8 = (uint32_t)__builtin_amdgcn_sbfe((int)r, 3, 1), m16 = (uint32_t)__builtin_amdgcn_sbfe((int)r, 4, 1);
        const uint32_t d0 = mask_select(m16, mask_select(m8, w[0], w[1]), w[2]);
        const uint32_t d1 = mask_select(m16, mask_select(m8, w[1], w[2]), w[3]);
        const uint32_t d2 = mask_select(m8, w[2], w[3]) & ~m16;
        win[2] = __builtin_amdgcn_alignbit(d1, d0, r * 4u);
        const uint32_t h1 = __builtin_amdgcn_alignbit(d2, d1, r * 4u);
        win[3] = (uint32_t)((((uint64_t)h1 << 32) | win[2]) >> (4u * (rk[3] - rk[2])));
      }
      const uint32_t nz = 0x80808080u - perm(0u, zs[ci], 0x00000000u);      // (the zero point in every byte)
      v4i acc[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) acc[g] = (v4i){0, 0, 0, 0};
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint32_t bfrag[4];
#pragma unroll
        for (int jj2 = 0; jj2 < 2; ++jj2) {
          const int jj = 2 * half + jj2;
          const uint32_t p0 = bias_pool(win[jj] & 0x0F0F0F0Fu, nz), p1 = bias_pool((win[jj] >> 4) & 0x0F0F0F0Fu, nz);
          bfrag[2 * jj2] = perm(p1, p0, sel[jj].x);                 // q - zero of columns 0-3 of the mask byte; pruned: 0
          bfrag[2 * jj2 + 1] = perm(p1, p0, sel[jj].y);             // columns 4-7
        }
        const v4i bv = (v4i){(int)bfrag[0], (int)bfrag[1], (int)bfrag[2], (int)bfrag[3]};
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const v4i av = *(const v4i*)(smem + aaddr[g] + 16 * half);
          acc[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[g], 0, 0, 0);
          asm("s_nop 1" : "+v"(acc[g]));                            // as in the kernels above
        }
      }
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const float dl = delta[dm[g] * (NCH + 4) + chunk];          // 0 past the last chunk
        const float f = fmaf((float)(acc[g][0] * 256 + acc[g][1]), 256.f, (float)acc[g][2]);
        ysum[4 * g + ci] = fmaf(f, h2f((uint16_t)(zs[ci] >> 8)) * dl, ysum[4 * g + ci]);
      }
    }
    if (BAR && S + 1 == s1) {                                       // the item is done: every wavefront meets at the barrier
      float* rb = red + (size_t)(p.round & 1) * M * 256;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int q = 4 * g;
        const float ps = (ysum[q] + ysum[q + 1]) + (ysum[q + 2] + ysum[q + 3]);
        if (kq + 4 * g < M) rb[((kq + 4 * g) * 16 + wave) * 16 + wr] = ps;
#pragma unroll
        for (int i = 0; i < 4; ++i) ysum[q + i] = 0.f;
      }
      __syncthreads();
      finish_round(p.round);
    }
    if (SPLIT && S + 1 == s1 && live) {                             // the item is done: its sums go to the caller's buffer
      const int tile = T_lo + p.round * TPR + tir;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int q = 4 * g;
        const float ps = (ysum[q] + ysum[q + 1]) + (ysum[q + 2] + ysum[q + 3]);
        if (kq + 4 * g < M) a.part[(((size_t)tile * a.sk + part) * M + kq + 4 * g) * 16 + wr] = ps;
#pragma unroll
        for (int i = 0; i < 4; ++i) ysum[q + i] = 0.f;
      }
    }
    if (!BAR && !SPLIT && S + 1 == s1 && live) {                    // the item is done
      // Lane quarter kq holds the sums of activation rows kq and 4 + kq.  The parts of a tile meet
      // in LDS, in the buffer of the round's parity, and the wavefront that arrives last adds them
      // in part order (not arrival order).  No barrier: a wavefront may be rounds ahead of the
      // others of its tile, so before it writes into a buffer it waits until the sums of the
      // round that used the buffer last have been added (by a wavefront that waits for nobody
      // who is behind it: all of them arrived at that round before this one could get here).
      const int tile = T_lo + p.round * TPR + tir;
      float ps[NG];
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int q = 4 * g;
        ps[g] = (ysum[q] + ysum[q + 1]) + (ysum[q + 2] + ysum[q + 3]);
#pragma unroll
        for (int i = 0; i < 4; ++i) ysum[q + i] = 0.f;
      }
      if (SK == 1) {
#pragma unroll
        for (int g = 0; g < NG; ++g)
          if (kq + 4 * g < M) store(kq + 4 * g, tile, ps[g]);
      } else {
        float* rb = red + (size_t)(p.round & 1) * M * 256;
        if (p.round >= 2)
          while (__hip_atomic_load(&summed[tir], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < p.round - 1)
            __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int g = 0; g < NG; ++g)
          if (kq + 4 * g < M) rb[((kq + 4 * g) * 16 + wave) * 16 + wr] = ps[g];
        // release: this wavefront's sums are in LDS before its arrival is counted; acquire: the
        // last one reads the others' sums only after it has seen all their arrivals
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        int old = 0;
        int* const arr = &arrived[(p.round & 1) * GV_WAVES + tir];   // (the next round counts in the other one; the one
        if (lane == 0) old = atomicAdd(arr, 1);                     //  after it starts only when this one is back at zero)
        old = __builtin_amdgcn_readfirstlane(old);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        if (old == SK - 1) {                                        // uniform over the wavefront
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            const int am = kq + 4 * g;
            if (am < M) {
              float v = 0.f;                                        // (four at a time; parts past SK re-read the last one and do not count)
              for (int j0 = 0; j0 < SK; j0 += 4) {
                float pv[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) pv[j] = rb[(am * 16 + tir * SK + (j0 + j < SK ? j0 + j : SK - 1)) * 16 + wr];
#pragma unroll
                for (int j = 0; j < 4; ++j) v += j0 + j < SK ? pv[j] : 0.f;
              }
              store(am, tile, v);
            }
          }
          if (lane == 0) *arr = 0;
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");          // the sums have been read, the counter is back at zero
          if (lane == 0) __hip_atomic_store(&summed[tir], p.round + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
    }
  };

  // ---- the first loads (row offsets, then mask words), then selector table and activation digits
  Pos pc{0, s0, m_row_off[row_of(tile_of(0))]};
  SmMask mk;
  SmCodes ca, cb;                                                  // swap roles by name (a copy would wait for the loads)
  issue_mask(pc, mk);
  if (tid < 256) {
    const uint2 e = make_selectors((uint32_t)tid, 0);
#pragma unroll
    for (int j = 0; j < LUT_LANES; ++j) lut[tid * LUT_LANES + j] = e;
  } else if (tid < 256 + (ZERO_BYTES + CNT_BYTES) / 4) {
    ((uint32_t*)zreg)[tid - 256] = 0u;                             // zero row and counters
  } else if (SPLIT && tid < 256 + (ZERO_BYTES + CNT_BYTES) / 4 + 4 * M) {       // deltas of the chunks past N
    const int i = tid - 256 - (ZERO_BYTES + CNT_BYTES) / 4;
    delta[(i >> 2) * (NCH + 4) + NCH + (i & 3)] = 0.f;
  }
  const int n16 = cols >> 4, xitems = M * n16;                     // a multiple of 8
  for (int it = tid; it < xitems; it += GV_THREADS) {
    XLoad xl;
    stage_load(a.x, a.ldx, m.cs, N, col0, n16, it, false, a.par, xl);
    stage_convert<0>(xl, m.cs != nullptr, a.xdt, N, ch0, n16, it, false, xq, delta, X_PAD);
  }
  __syncthreads();
  if (idle) {                                                      // (uniform over the wavefront) no item
    if (BAR)
      for (int round = 0; round < R; ++round) {
        __syncthreads();
        finish_round(round);
      }
    return;
  }
  issue_codes(pc, mk, ca);
  Pos pb = pc;                                                     // position whose codes are fetched next
  advance(pb);
  issue_mask(pb, mk);
  Pos pa = pb;                                                     // position whose mask words are being fetched
  const int total = R * (s1 - s0);
  for (int q = 0; q < total; q += 2) {
    issue_codes(pb, mk, cb);
    advance(pa);
    issue_mask(pa, mk);
    compute(pc, ca);
    pc = pb; pb = pa;
    if (q + 1 >= total) break;
    issue_codes(pb, mk, ca);
    advance(pa);
    issue_mask(pa, mk);
    compute(pc, cb);
    pc = pb; pb = pa;
  }
}

constexpr int STREAM_MFMA_MIN_STEPS = 1536;     // tile-steps (16 rows x 512 columns) from which the matrix-core kernel is used

template <int NG, bool BAR, bool SPLIT = false>
static int launch_stream_mfma_ng(const SmArgs& a, size_t lds, int blocks, hipStream_t st) {
  auto kern = gemv_stream_mfma_kernel<NG, BAR, SPLIT>;
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(GV_THREADS), lds, st, a);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

// LDS of the kernel for mp activation rows of N columns
static inline size_t stream_mfma_lds(int N, int mp) {
  return (size_t)LUT_BYTES + ZERO_BYTES + CNT_BYTES + (size_t)mp * NDIG * (N + X_PAD) + (size_t)mp * (N / 128 + 4) * 4 + (size_t)2 * mp * 256 * 4;
}

// What the matrix-core stream kernel does with a matrix: false if it is not one of its cases.
// By the shape alone: which kernel runs, and how a row is cut into parts, must not depend on M,
// or a row's result would.
struct SmPlan { int ntiles, blocks, tq, tr, nS, sk, spi, mc; };
static bool stream_mfma_plan(const DMat& m, SmPlan& p) {
  if (m.layout != CBK_SPARSE4X && m.layout != CBK_SPARSE4E) return false;
  if (m.N % 128 != 0 || m.K < 1) return false;
  p.mc = GV_MAX_M;                                                  // activation rows per pass of whole rows: what fits in LDS
  while (p.mc > 0 && stream_mfma_lds(m.N, p.mc) > (size_t)160 * 1024) --p.mc;
  if (p.mc == 0) return false;
  p.ntiles = (m.K + 15) / 16;
  p.nS = (m.N / 128 + 3) / 4;
  // Small matrices stay on the row kernel, which is faster there at one activation row
  // (4096 x 2048, 1024 tile-steps: 6.6 against 8.3 us; 2048 x 4096: 8.4 against 8.8 us, but 12.2
  // against 10.1 us at M = 4; 4096 x 4096, 2048 tile-steps: 8.8 / 13.0 / 19.4 us at M = 1 / 4 / 8
  // against 9.2 / 10.7 / 15.1 us here; 1024 x 14336, 1792: 17.8 against 15.7 us at M = 1).
  if ((long long)p.ntiles * p.nS < STREAM_MFMA_MIN_STEPS) return false;
  p.blocks = p.ntiles < 256 ? p.ntiles : 256;                       // one persistent workgroup per CU
  p.tq = p.ntiles / p.blocks; p.tr = p.ntiles % p.blocks;
  // Parts per tile: as few steps per wavefront as possible, and few tiles per round.  With one
  // or two tiles in a round the sixteen wavefronts read the same 16 or 32 rows side by side: the
  // cache lines of their offsets, scales and zero points (64 groups or more each) and of their
  // mask words and codes serve several wavefronts before they are displaced, and a step is
  // 15-25 % faster (65536 x 4096 at M = 1: 49.0 us with sixteen tiles in one round, 44.1 us with
  // two in each of eight rounds; 32768 x 8192: 49.8 / 49.0 / 45.2 us with eight / two / one).  A
  // round costs about an eighth of a step beside its steps.  No part may be empty.
  const int tmax = p.tq + (p.tr ? 1 : 0);
  float best = 0.f;
  p.sk = 1; p.spi = p.nS;
  for (int sk = 1; sk <= GV_WAVES && sk <= p.nS; ++sk) {
    const int spi = (p.nS + sk - 1) / sk;
    if ((sk - 1) * spi >= p.nS) continue;
    const int tpr = GV_WAVES / sk, rounds = (tmax + tpr - 1) / tpr;
    const float c = (float)rounds * ((float)spi * (tpr == 1 ? 0.75f : tpr == 2 ? 0.85f : 1.f) + 0.12f);
    if (sk == 1 || c < best) { best = c; p.sk = sk; p.spi = spi; }
  }
  return true;
}

// The q | k | v ranges of a survivor-stream matrix with three col_scale vectors, each as a matrix
// with one vector (the rows of such a matrix are found through row_off, so any row starts a
// range).  Returns how many are not empty.
static int stream_row_ranges(const DMat& m, DMat (&sub)[3], int (&lo)[3]) {
  const int b0 = m.cs_split0, b1 = m.cs_split0 + m.cs_split1;
  const int l[3] = {0, b0, b1}, h[3] = {b0, b1, m.K};
  int n = 0;
  for (int r = 0; r < 3; ++r) {
    if (h[r] <= l[r]) continue;
    DMat d = m;
    d.row_off = m.row_off + l[r];
    d.scale = m.scale + (size_t)l[r] * m.G;
    d.zero = m.zero + (size_t)l[r] * m.G;
    d.K = h[r] - l[r];
    d.cs = m.cs + (size_t)r * m.N;
    d.cs_rows = 1;
    d.cs_split0 = d.cs_split1 = 0;
    sub[n] = d; lo[n] = l[r];
    ++n;
  }
  return n;
}

// Room for the part sums of a call whose activation rows do not fit in LDS as whole rows; 0: none needed.
size_t gemv_stream_workspace(const DMat& m, int M) {
  if (family_of(m.layout) == FAM_SPARSE && m.cs_rows == 3 && m.cs) {   // run range by range, on the same bytes
    DMat sub[3];
    int lo[3];
    size_t need = 0;
    const int n = stream_row_ranges(m, sub, lo);
    for (int i = 0; i < n; ++i) {
      const size_t b = gemv_stream_workspace(sub[i], M);
      need = need > b ? need : b;
    }
    return need;
  }
  SmPlan p;
  if (family_of(m.layout) != FAM_SPARSE || m.bits != 4 || m.group != 128 || m.cs_rows > 2) return 0;
  const int vm = m.cs_rows == 2 ? 2 : 1;
  const int Ms = M * vm < GV_MAX_M ? M * vm : GV_MAX_M;              // kernel rows of a pass over the weights
  if (!(m.flags & CBK_FLAG_ZERO_LE_128) || !stream_mfma_plan(m, p) || Ms <= p.mc || p.sk < 2) return 0;
  return up256(split_part_bytes(p.ntiles, p.sk, Ms));
}

// CBK_ERR_UNSUPPORTED: not a case of this kernel.
static int launch_gemv_stream_mfma(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                                   const void* bias, void* ws, size_t ws_bytes, hipStream_t st) {
  SmPlan p;
  if (!stream_mfma_plan(m, p)) return CBK_ERR_UNSUPPORTED;
  SmArgs a;
  a.m = m; a.ldx = ldx; a.ldy = ldy; a.bias = bias; a.xdt = xdt; a.ydt = ydt;
  a.ntiles = p.ntiles; a.tq = p.tq; a.tr = p.tr; a.nS = p.nS; a.sk = p.sk; a.spi = p.spi;
  a.hdr = ((m.N >> 3) + ((m.G * 2 + 15) & ~15) + 15) & ~15;
  a.inv_sk = (uint32_t)((65536 + a.sk - 1) / a.sk);
  a.pps = a.sk; a.wps = p.blocks; a.part = nullptr;
  // a fused gate/up matrix (two col_scale vectors by row parity) stages two scaled copies of every activation row
  const int vm = m.cs_rows == 2 ? 2 : 1;
  a.par = vm == 2 ? 1 : 0;
  if (p.mc < vm) return CBK_ERR_UNSUPPORTED;
  const size_t ysz = ydt == CBK_F32 ? 4 : 2;
  // More activation rows than fit in LDS as whole rows: with room for the part sums the
  // workgroups split the row by columns (whole parts: the same parts, added in the same order by
  // the reduce kernel of the column-split path above, so the same bits), up to eight activation
  // rows per pass over the weights; without it the rows go in passes of what fits.
  const int Ms = M * vm < GV_MAX_M ? M * vm : GV_MAX_M;              // kernel rows of a pass
  if (Ms > p.mc && p.sk >= 2 && ws && !((uintptr_t)ws & 15) && ws_bytes >= split_part_bytes(p.ntiles, p.sk, Ms)) {
    const size_t fixed = (size_t)LUT_BYTES + ZERO_BYTES + CNT_BYTES + (size_t)Ms * (m.N / 128 + 4) * 4 + (size_t)Ms * NDIG * X_PAD;
    const size_t per_part = (size_t)Ms * NDIG * p.spi * 512;
    int pps_max = fixed < (size_t)160 * 1024 ? (int)(((size_t)160 * 1024 - fixed) / per_part) : 0;
    pps_max = pps_max < p.sk ? pps_max : p.sk;
    if (pps_max >= 1) {
      // parts per slab: rounds of one part per wavefront after staging the slab (a 512-column
      // step of eight rows costs about 0.15 rounds of one step to stage)
      float best = 0.f;
      int best_pps = 0, best_wps = 1;
      for (int pps = 1; pps <= pps_max; ++pps) {
        const int nslab = (p.sk + pps - 1) / pps;
        if (nslab > 256) continue;
        int wps = 256 / nslab;
        wps = wps > p.ntiles ? p.ntiles : wps;
        const int tpw = (p.ntiles + wps - 1) / wps, tpr = GV_WAVES / pps;
        const float c = (float)((tpw + tpr - 1) / tpr * p.spi) + 0.15f * (float)Ms / 8.f * (float)(pps * p.spi);
        if (best_pps == 0 || c < best) { best = c; best_pps = pps; best_wps = wps; }
      }
      if (best_pps > 0) {
        const int nslab = (p.sk + best_pps - 1) / best_pps;
        a.pps = best_pps; a.wps = best_wps;
        a.tq = p.ntiles / best_wps; a.tr = p.ntiles % best_wps;
        a.part = (float*)ws;
        const size_t lds = fixed + (size_t)Ms * NDIG * best_pps * p.spi * 512;
        GsArgs r = {};                                                // the reduce launch: one matrix
        r.h.n = 1; r.h.ydt = ydt; r.h.xdt = xdt; r.h.xq_cap = 0; r.h.delta_cap = 0;
        for (int i = 0; i < GV_MAX_BATCH; ++i) { r.h.wg_end[i] = 0x7fffffff; r.h.th_end[i] = 0x7fffffff; }
        GsMat& q = r.mat[0];
        q.g.m = m; q.g.par = a.par; q.g.bias = bias; q.g.ldy = ldy; q.g.ntiles = p.ntiles; q.g.sk = p.sk;
        q.th0 = 0; q.wg0 = 0; q.part = (float*)ws;
        for (int m0 = 0; m0 < M; m0 += GV_MAX_M / vm) {
          const int mp = (M - m0 < GV_MAX_M / vm ? M - m0 : GV_MAX_M / vm) * vm;      // kernel rows
          a.x = (const uint16_t*)x + (size_t)m0 * ldx;
          a.M = mp;
          const int rc = mp > 4 ? launch_stream_mfma_ng<2, false, true>(a, lds, nslab * best_wps, st)
                                : launch_stream_mfma_ng<1, false, true>(a, lds, nslab * best_wps, st);
          if (rc) return rc;
          r.h.M = mp;
          q.g.y = (uint8_t*)y + (size_t)m0 * ldy * ysz;
          const int th = (p.ntiles * mp * 16 + GS_RED_THREADS - 1) / GS_RED_THREADS * GS_RED_THREADS;
          r.h.th_end[0] = th;
          hipLaunchKernelGGL(gemv_split_reduce_kernel, dim3(th / GS_RED_THREADS), dim3(GS_RED_THREADS), 0, st, r);
          if (hipGetLastError() != hipSuccess) return CBK_ERR_HIP;
        }
        return CBK_OK;
      }
    }
  }
  const int mr = p.mc / vm;                                             // activation rows that fit
  const int mc = (M + (M + mr - 1) / mr - 1) / ((M + mr - 1) / mr);     // as few passes as fit, of equal size
  for (int m0 = 0; m0 < M; m0 += mc) {
    const int mp = (M - m0 < mc ? M - m0 : mc) * vm;                    // kernel rows
    a.x = (const uint16_t*)x + (size_t)m0 * ldx;
    a.y = (uint8_t*)y + (size_t)m0 * ldy * ysz;
    a.M = mp;
    const size_t lds = stream_mfma_lds(m.N, mp);
    // One activation row: the round ends in a barrier; more: arrival counters (the same sums in
    // the same order either way).  65536 x 4096, us per call with barrier / counters: M = 1
    // 42.4 / 44.3, M = 2 44.4 / 44.4, M = 3 47.4 / 44.8, M = 4 49.1 / 45.6, M = 8 62 / 51.
    const int rc = mp > 4 ? launch_stream_mfma_ng<2, false>(a, lds, p.blocks, st)
                 : mp == 1 ? launch_stream_mfma_ng<1, true>(a, lds, p.blocks, st) : launch_stream_mfma_ng<1, false>(a, lds, p.blocks, st);
    if (rc) return rc;
  }
  return CBK_OK;
}

// CBK_ERR_UNSUPPORTED: not a case of this kernel (the caller falls back on the float row kernel).
int launch_gemv_stream(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                       const void* bias, void* ws, size_t ws_bytes, hipStream_t st) {
  if (family_of(m.layout) != FAM_SPARSE || m.bits != 4 || m.group != 128 || m.cs_rows > 3) return CBK_ERR_UNSUPPORTED;
  if (!(m.flags & CBK_FLAG_ZERO_LE_128)) return CBK_ERR_UNSUPPORTED;
  if (xdt != CBK_F16 && xdt != CBK_BF16T) return CBK_ERR_DTYPE;
  if (m.cs_rows == 3) {
    // a fused q | k | v matrix: its three row ranges one after the other, each with its own
    // col_scale vector (and, by its own shape, on the matrix-core or on the row kernel)
    if (!m.cs || (size_t)NDIG * m.N > (size_t)ST_X_BUDGET) return CBK_ERR_UNSUPPORTED;
    DMat sub[3];
    int lo[3];
    const int n = stream_row_ranges(m, sub, lo);
    const size_t ysz = ydt == CBK_F32 ? 4 : 2;
    for (int i = 0; i < n; ++i) {
      const int rc = launch_gemv_stream(sub[i], x, xdt, M, ldx, (uint8_t*)y + (size_t)lo[i] * ysz, ydt, ldy,
                                        bias ? (const uint8_t*)bias + (size_t)lo[i] * ysz : nullptr, ws, ws_bytes, st);
      if (rc) return rc;
    }
    return CBK_OK;
  }
  {
    const int rc = launch_gemv_stream_mfma(m, x, xdt, M, ldx, y, ydt, ldy, bias, ws, ws_bytes, st);   // the layouts with group offsets
    if (rc != CBK_ERR_UNSUPPORTED) return rc;
  }
  if (m.cs_rows > 1) return CBK_ERR_UNSUPPORTED;                     // (fused gate/up: the matrix-core kernel only)
  if ((size_t)NDIG * m.N > (size_t)ST_X_BUDGET) return CBK_ERR_UNSUPPORTED;
  int mc = (int)((size_t)ST_X_BUDGET / ((size_t)NDIG * m.N));      // activation rows per pass
  mc = mc > ST_MAX_M ? ST_MAX_M : mc;
  for (int m0 = 0; m0 < M; m0 += mc) {
    const int mp = M - m0 < mc ? M - m0 : mc;
    const void* xs = (const uint8_t*)x + (size_t)m0 * ldx * 2;
    void* ys = (uint8_t*)y + (size_t)m0 * ldy * (ydt == CBK_F32 ? 4 : 2);
    int rc;
    switch (mp) {
      case 1: rc = launch_stream_m<1>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 2: rc = launch_stream_m<2>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 3: rc = launch_stream_m<3>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 4: rc = launch_stream_m<4>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 5: rc = launch_stream_m<5>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 6: rc = launch_stream_m<6>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 7: rc = launch_stream_m<7>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      default: rc = launch_stream_m<8>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
    }
    if (rc) return rc;
  }
  return CBK_OK;
}

// ------------------------------------------------------------------ 8-bit dense rows
// DENSE8 (group 128) at one to eight activation rows per pass, on the same activation digits:
// the codes are the bytes themselves, q - 128 is a signed byte (one xor), and
//   sum_j (q_j - z) X_j = sum_j (q_j - 128) X_j - (z - 128) sum_j X_j
// with the integer activations X of the group; their sum per 128-column chunk is formed once per
// launch from the digits.  One wavefront per weight row, one lane per 32-column block (32 code
// bytes), v_dot4_i32_i8 per four columns and digit, the next block's loads in flight while this
// one is multiplied.  Any uint8 zero point.
// Reference semantics: cbk::detail::gemv_dense8 (src/cobaltkernel/csrc/cobalt_gemv.cuh:1127-1171).
struct D8Loads { uint4 c0, c1; uint32_t sraw, z; };

template <int M>
__global__ __launch_bounds__(ST_THREADS) void gemv_dense8_kernel(DMat m, const uint16_t* x, int64_t ldx, int xdt,
                                                                 void* y, int ydt, int64_t ldy, const void* bias) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int N = m.N, NCH = N >> 7, NB = N >> 5;
  int8_t* xq = (int8_t*)smem;
  float* delta = (float*)(xq + (size_t)M * NDIG * N);
  float* fsum = delta + M * (NCH + 4);                            // [M][NCH] sum of the chunk's integer activations
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // this wavefront's rows kw, kw + ks, ...; its items are (row, pass over the row's blocks), in order
  // (a wavefront without rows goes through the first loads on the last row and leaves after the barriers)
  const int kw = (int)blockIdx.x * ST_WAVES + wave, ks = (int)gridDim.x * ST_WAVES;
  const int k0 = kw < m.K ? kw : m.K - 1;
  const int nrows = kw < m.K ? (m.K - k0 + ks - 1) / ks : 0;
  const int nt = (NB + 63) >> 6, nitems = nrows * nt;
  struct Pos { int k, it; };
  auto next_pos = [&](Pos& p) {
    if (p.it + 1 < nt) { ++p.it; return; }
    if (p.k + ks < m.K) { p.k += ks; p.it = 0; }
  };
  auto issue = [&](const Pos& p, D8Loads& L) {
    int t = lane + 64 * p.it;
    t = t < NB ? t : NB - 1;
    const RowView row = row_view(m, p.k);
    L.c0 = *(const uint4*)row.unit(2 * t);
    L.c1 = *(const uint4*)row.unit(2 * t + 1);
    const size_t gi = meta_index(m, p.k, t >> 2);
    L.sraw = m.scale[gi];
    L.z = m.zero[gi];
  };
  float ysum[M];
#pragma unroll
  for (int i = 0; i < M; ++i) ysum[i] = 0.f;
  auto compute = [&](const Pos& p, const D8Loads& L) {
    const int traw = lane + 64 * p.it;
    const bool valid = traw < NB;
    const int t = valid ? traw : NB - 1, g = t >> 2;
    const uint32_t cw[8] = {L.c0.x, L.c0.y, L.c0.z, L.c0.w, L.c1.x, L.c1.y, L.c1.z, L.c1.w};
    int acc[M][NDIG];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
      for (int d = 0; d < NDIG; ++d) acc[i][d] = 0;
    // the lanes take the two 16-byte halves of their blocks in alternating order: the digits of
    // neighbouring lanes are 32 bytes apart, and sixteen 16-byte reads at that stride would fall
    // on half of the LDS banks
    const int rot = (lane >> 3) & 1;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int hh = h ^ rot;
      uint32_t b[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) b[u] = (hh ? cw[4 + u] : cw[u]) ^ 0x80808080u;      // q - 128 as signed bytes
#pragma unroll
      for (int i = 0; i < M; ++i)
#pragma unroll
        for (int d = 0; d < NDIG; ++d) {
          const uint4 a = *(const uint4*)(xq + (size_t)(i * NDIG + d) * N + t * 32 + 16 * hh);
          acc[i][d] = __builtin_amdgcn_sdot4((int)b[0], (int)a.x, acc[i][d], false);
          acc[i][d] = __builtin_amdgcn_sdot4((int)b[1], (int)a.y, acc[i][d], false);
          acc[i][d] = __builtin_amdgcn_sdot4((int)b[2], (int)a.z, acc[i][d], false);
          acc[i][d] = __builtin_amdgcn_sdot4((int)b[3], (int)a.w, acc[i][d], false);
        }
    }
    const float s = valid ? h2f((uint16_t)L.sraw) : 0.f;
    const float zc = (t & 3) == 0 ? (float)((int)L.z - 128) : 0.f;   // the group's zero-point term: once, in its first block
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const float f = fmaf((float)(acc[i][0] * 256 + acc[i][1]), 256.f, (float)acc[i][2]);
      ysum[i] = fmaf(fmaf(-zc, fsum[i * NCH + g], f), s * delta[i * (NCH + 4) + g], ysum[i]);
    }
    if (p.it + 1 == nt) {                                         // the row is complete
      const int k = p.k;
#pragma unroll
      for (int i = 0; i < M; ++i) {
        const float v0 = ysum[i];
        ysum[i] = 0.f;
        float v = wave_sum_dpp(v0);
        if (lane == 0) {
          if (bias) v += (ydt == CBK_F32) ? ((const float*)bias)[k]
                       : (ydt == CBK_F16) ? h2f(((const uint16_t*)bias)[k]) : bf2f(((const uint16_t*)bias)[k]);
          if (ydt == CBK_F32) ((float*)y)[(size_t)i * ldy + k] = v;
          else if (ydt == CBK_F16) ((uint16_t*)y)[(size_t)i * ldy + k] = f2h(v);
          else ((uint16_t*)y)[(size_t)i * ldy + k] = f2bf(v);
        }
      }
    }
  };

  Pos pc{k0, 0};                                                  // item being multiplied
  D8Loads la, lb;                                                 // swap roles by name (a copy would wait for the loads)
  issue(pc, la);
  Pos pn = pc;                                                    // item whose bytes are being fetched
  next_pos(pn);
  // activation digits and the chunks' sums, while the first row's bytes are on their way
  const int n16 = N >> 4, xitems = M * n16;                      // a multiple of 8
  for (int it = tid; it < xitems; it += ST_THREADS) {
    XLoad xl;
    stage_load(x, ldx, m.cs, N, 0, n16, it, M == 1, 0, xl);
    stage_convert<0>(xl, m.cs != nullptr, xdt, N, 0, n16, it, M == 1, xq, delta);
  }
  __syncthreads();
  for (int c = tid; c < M * NCH; c += ST_THREADS) {
    const int row = c / NCH, ch = c - row * NCH;
    int sd[NDIG];
#pragma unroll
    for (int d = 0; d < NDIG; ++d) {
      int sum = 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const uint4 a = *(const uint4*)(xq + (size_t)(row * NDIG + d) * N + ch * 128 + 16 * u);
        sum = __builtin_amdgcn_sdot4(0x01010101, (int)a.x, sum, false);
        sum = __builtin_amdgcn_sdot4(0x01010101, (int)a.y, sum, false);
        sum = __builtin_amdgcn_sdot4(0x01010101, (int)a.z, sum, false);
        sum = __builtin_amdgcn_sdot4(0x01010101, (int)a.w, sum, false);
      }
      sd[d] = sum;
    }
    fsum[c] = (float)((sd[0] * 256 + sd[1]) * 256 + sd[2]);       // |sum| < 2^31: 128 columns of at most 127 * 65536
  }
  __syncthreads();
  if (kw >= m.K) return;
  for (int q = 0; q < nitems; q += 2) {
    issue(pn, lb);
    compute(pc, la);
    pc = pn; next_pos(pn);
    if (q + 1 >= nitems) break;
    issue(pn, la);
    compute(pc, lb);
    pc = pn; next_pos(pn);
  }
}

template <int M>
static int launch_dense8_m(const DMat& m, const void* x, int64_t ldx, int xdt, void* y, int ydt, int64_t ldy,
                           const void* bias, hipStream_t st) {
  auto kern = gemv_dense8_kernel<M>;
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  const size_t lds = (size_t)M * NDIG * m.N + (size_t)M * (m.N / 128 + 4) * 4 + (size_t)M * (m.N / 128) * 4;
  if (lds > 160 * 1024) return CBK_ERR_UNSUPPORTED;
  int blocks = (m.K + ST_WAVES - 1) / ST_WAVES;
  blocks = blocks < 256 ? blocks : 256;                           // one persistent workgroup per CU
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(ST_THREADS), lds, st, m, (const uint16_t*)x, ldx, xdt, y, ydt, ldy, bias);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

// CBK_ERR_UNSUPPORTED: not a case of this kernel (the caller falls back on the float row kernel).
int launch_gemv_dense8(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                       const void* bias, hipStream_t st) {
  if (m.layout != CBK_DENSE8 || m.bits != 8 || m.group != 128 || m.cs_rows > 1) return CBK_ERR_UNSUPPORTED;
  if (xdt != CBK_F16 && xdt != CBK_BF16T) return CBK_ERR_DTYPE;
  if ((size_t)NDIG * m.N > (size_t)ST_X_BUDGET) return CBK_ERR_UNSUPPORTED;
  int mc = (int)((size_t)ST_X_BUDGET / ((size_t)NDIG * m.N));      // activation rows per pass
  mc = mc > ST_MAX_M ? ST_MAX_M : mc;
  for (int m0 = 0; m0 < M; m0 += mc) {
    const int mp = M - m0 < mc ? M - m0 : mc;
    const void* xs = (const uint8_t*)x + (size_t)m0 * ldx * 2;
    void* ys = (uint8_t*)y + (size_t)m0 * ldy * (ydt == CBK_F32 ? 4 : 2);
    int rc;
    switch (mp) {
      case 1: rc = launch_dense8_m<1>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 2: rc = launch_dense8_m<2>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 3: rc = launch_dense8_m<3>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 4: rc = launch_dense8_m<4>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 5: rc = launch_dense8_m<5>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 6: rc = launch_dense8_m<6>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      case 7: rc = launch_dense8_m<7>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
      default: rc = launch_dense8_m<8>(m, xs, ldx, xdt, ys, ydt, ldy, bias, st); break;
    }
    if (rc) return rc;
  }
  return CBK_OK;
}

// ------------------------------------------------------------------ host side

static bool keep_supported(int keep) { return keep == 10 || keep == 16 || keep == 23; }

bool gemv_fast_takes(const DMat& m, int M) {
  if (M < 1 || M > GV_MAX_M) return false;
  if (M > 4 && !block_split_capable(m.bits, family_of(m.layout) == FAM_DENSE ? 0 : m.keep, m.group)) return false;
  if (m.cs_rows == 3) return false;                              // the caller splits q|k|v into its ranges
  if (!(m.flags & CBK_FLAG_ZERO_LE_128)) return false;
  const int fam = family_of(m.layout);
  if (fam == FAM_BLK) { if (!keep_supported(m.keep)) return false; }
  else if (fam == FAM_DENSE) { if (m.bits == 8) return false; }
  else if (fam == FAM_BLK6) { if (m.bits != 6 || m.keep != 16 || m.group != 128) return false; }
  else return false;
  if (m.bits != 2 && m.bits != 3 && m.bits != 4 && fam != FAM_BLK6) return false;
  // 32-bit offsets inside the kernel: every array of the matrix below 4 GB
  if ((uint64_t)((m.K + 15) / 16 * 16) * m.stride + 1024 >= (1ull << 32)) return false;
  if ((uint64_t)((m.K + 15) / 16 * 16) * m.G * 2 >= (1ull << 32)) return false;
  // the digits are staged in column slabs where a whole row does not fit; the per-chunk deltas
  // of all rows stay in LDS for the whole matrix
  if (M == 1) return (size_t)NDIG * (m.N + X_PAD) <= (size_t)X_LDS_BUDGET;   // (the one-row kernels stage whole rows only)
  return (size_t)M * (m.N / 128 + 4) * 4 <= (size_t)DELTA_LDS_BUDGET;
}

bool gemv_same_config(const DMat& a, const DMat& b) {
  const bool da = family_of(a.layout) == FAM_DENSE, db = family_of(b.layout) == FAM_DENSE;
  return da == db && a.bits == b.bits && a.group == b.group && (da || a.keep == b.keep);
}

// Macro-steps per work item of a launch of `cost` tile-steps on `blocks` workgroups: about one and
// a half items per wavefront over the whole launch (the end of an item costs about as many
// instructions as a step; measured best between one and two).
static inline int launch_spi(long long cost, int blocks) {
  const int spi = (int)(cost * 2 / ((long long)blocks * GV_WAVES * 3));
  return spi < 1 ? 1 : (spi > 8 ? 8 : spi);
}
// The parts of a row of nS macro-steps: at most 16, a power of two of them where the row is long
// enough (the items then spread evenly over the four SIMDs), of equal length.
static inline void row_parts(int nS, int spi_launch, int& spi, int& sk) {
  int s = spi_launch;
  while ((nS + s - 1) / s > 16) ++s;
  sk = (nS + s - 1) / s;
  int p2 = 1;
  while (p2 < sk) p2 <<= 1;
  if (p2 <= 16 && p2 <= nS) sk = p2;
  spi = (nS + sk - 1) / sk;
  sk = (nS + spi - 1) / spi;
}
// LDS left for the activation digits of M rows beside the selector table, the deltas and two
// reduction slots (up to 24 KB of slots where there is room)
static inline size_t main_x_budget(int M, int delta_cap, int sk_cap) {
  const size_t slot_bytes = (size_t)sk_cap * M * 16 * 4;
  const size_t fixed = (size_t)LUT_BYTES + ZERO_BYTES + CNT_BYTES + (size_t)delta_cap * 4;
  const size_t red_floor = 2 * slot_bytes < 24 * 1024 ? 2 * slot_bytes : 24 * 1024;
  return 160 * 1024 - fixed - red_floor;
}

// Rows whose digits (M * 3 * N bytes) stay within SPLIT_MIN_BYTES need no workspace; longer ones (two
// to eight activation rows of a block-per-quarter configuration) are split over the workgroups by
// columns when the caller provides room for the part sums: [tiles][parts <= 16][M][16] floats.
constexpr size_t SPLIT_MIN_BYTES = 90 * 1024;  // digits of a row (M * 3 * N bytes) from which it is split (measured on both layer sets
                                               // at 56, 72, 90 and 112 KB: six rows of 5376 and eight of 4096 columns gain, seven of 4096 lose)
constexpr int SPLIT_MAX_TILES = 4096;          // (rows that fit are split only in launches of at most this many tiles)
static inline int kernel_rows(const DMat& m, int M) {            // activation rows as the kernel counts them, per pass
  const int v = m.cs_rows == 2 ? 2 : 1;
  return M * v > GV_MAX_M ? GV_MAX_M : M * v;
}

size_t gemv_fast_workspace(const DMat& m, int M) {
  const int Mk = kernel_rows(m, M);
  if (Mk < 2 || !block_split_capable(m.bits, family_of(m.layout) == FAM_DENSE ? 0 : m.keep, m.group)) return 0;
  const size_t digits = (size_t)Mk * NDIG * (m.N + X_PAD);
  if (digits <= SPLIT_MIN_BYTES) return 0;
  // what a call with this matrix alone would do
  const int ntiles = (m.K + 15) / 16, nS = (m.N / 128 + 3) / 4;
  int spi, sk;
  row_parts(nS, launch_spi((long long)ntiles * nS, ntiles < 256 ? ntiles : 256), spi, sk);
  if (digits <= main_x_budget(Mk, Mk * (m.N / 128 + 4), sk) && ntiles > SPLIT_MAX_TILES) return 0;
  if (ntiles < 256) sk = nS < 16 ? nS : 16;                       // (in a batch a small matrix may be cut finer)
  return up256(split_part_bytes(ntiles + 3, sk, Mk));             // (+3: a q|k|v matrix is run as its three ranges)
}

struct GvCall {           // one matrix of a batched call, host side
  DMat m;
  const void* x;
  int64_t ldx;
  void* y;
  int64_t ldy;
  const void* bias;
  int par;                  // gate/up matrix: M counts real activation rows, the kernel sees 2 M
};

template <int BITS, int KEEP, int GRP, int MP>
static int launch_cfg(const GvBatch& b, size_t lds, int blocks, hipStream_t st) {
  auto kern = gemv_mfma_kernel<BITS, KEEP, GRP, MP>;
  static std::atomic<int> configured{0};
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(GV_THREADS), lds, st, b);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

template <int BITS, int KEEP, int GRP>
static int launch_mp(const GvBatch& b, size_t lds, int blocks, hipStream_t st) {
  if (b.h.M == 1) return launch_cfg<BITS, KEEP, GRP, 1>(b, lds, blocks, st);
  if constexpr (!block_split_capable(BITS, KEEP, GRP)) {
    if (b.h.M == 2) return launch_cfg<BITS, KEEP, GRP, 2>(b, lds, blocks, st);
  }
  if constexpr (block_split_capable(BITS, KEEP, GRP)) {
    if (b.h.M > 4) return launch_cfg<BITS, KEEP, GRP, 8>(b, lds, blocks, st);
  } else {
    if (b.h.M > 4) return CBK_ERR_UNSUPPORTED;
  }
  return launch_cfg<BITS, KEEP, GRP, 4>(b, lds, blocks, st);
}

template <int BITS, int KEEP>
static int launch_grp(const GvBatch& b, size_t lds, int blocks, hipStream_t st) {
  return b.mat[0].m.group == 64 ? launch_mp<BITS, KEEP, 64>(b, lds, blocks, st)
                                : launch_mp<BITS, KEEP, 128>(b, lds, blocks, st);
}

template <int BITS>
static int launch_keep(const GvBatch& b, size_t lds, int blocks, hipStream_t st) {
  const DMat& m = b.mat[0].m;
  switch (family_of(m.layout) == FAM_DENSE ? 0 : m.keep) {
    case 0: return launch_grp<BITS, 0>(b, lds, blocks, st);
    case 10: return launch_grp<BITS, 10>(b, lds, blocks, st);
    case 16: return launch_grp<BITS, 16>(b, lds, blocks, st);
    case 23: return launch_grp<BITS, 23>(b, lds, blocks, st);
    default: return CBK_ERR_UNSUPPORTED;
  }
}

// Workgroups of a launch of the main kernel.  A workgroup takes whole tiles.  Between one and two
// tiles per workgroup the launch lasts two tiles however they are dealt, and dealing two to each
// of fewer workgroups (384 tiles: 192 x 2 instead of 128 x 2 + 128 x 1) was measured faster as
// long as at least three quarters of the CUs still get one (Mistral q,k,v: -1.9 us); with fewer
// workgroups than that, or more tiles each, having every CU at work counts for more.  Only where
// every tile costs the same.
static int gemv_blocks(const GvBatch& gb, int n, int tiles) {
  int blocks = tiles < 256 ? tiles : 256;                       // one persistent workgroup per CU
  bool same = true;
  for (int i = 1; i < n; ++i) same = same && gb.mat[i].nS == gb.mat[0].nS;
  if (same && tiles > 256 && tiles <= 512 && (tiles + 1) / 2 >= 192) blocks = (tiles + 1) / 2;
  return blocks;
}

template <int BITS, int KEEP, int GRP, int MP>
static int launch_split_cfg(const GsArgs& a, size_t lds, int blocks, int red_blocks, hipStream_t st) {
  if constexpr ((MP == 4 || MP == 8) && block_split_capable(BITS, KEEP, GRP)) {
    auto kern = gemv_split_kernel<BITS, KEEP, GRP, MP>;
    static std::atomic<int> configured{0};
    if (!configured.load(std::memory_order_acquire)) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
        return CBK_ERR_HIP;
      configured.store(1, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(GV_THREADS), lds, st, a);
    if (hipGetLastError() != hipSuccess) return CBK_ERR_HIP;
    hipLaunchKernelGGL(gemv_split_reduce_kernel, dim3(red_blocks), dim3(GS_RED_THREADS), 0, st, a);
    return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
  } else {
    return CBK_ERR_UNSUPPORTED;
  }
}

// The matrices `mats` (spi and sk set) through one launch of gemv_split_kernel and one of the
// reduce kernel: workgroups per matrix by its share of the work, parts per slab, workgroups per
// slab, LDS.  `ws` holds the part sums of the matrices one after the other, each
// up256(split_part_bytes(ntiles, sk, M)).
static int launch_split_batch(const GvMat* mats, int n, int M, int xdt, int ydt, uint8_t* ws, hipStream_t st) {
  GsArgs a;
  a.h.n = n; a.h.M = M; a.h.xdt = xdt; a.h.ydt = ydt;
  long long total = 0;
  int delta_cap = 0;
  for (int i = 0; i < n; ++i) {
    total += (long long)mats[i].ntiles * mats[i].nS;
    delta_cap = delta_cap > M * (mats[i].m.N / 128 + 4) ? delta_cap : M * (mats[i].m.N / 128 + 4);
  }
  const size_t fixed = (size_t)LUT_BYTES + ZERO_BYTES + (size_t)delta_cap * 4 + (size_t)M * NDIG * X_PAD;
  int xq_cap = 0, wg = 0, th = 0;
  size_t off = 0;
  for (int i = 0; i < n; ++i) {
    GsMat& q = a.mat[i];
    const GvMat& g = mats[i];
    q.g = g;
    q.part = (float*)(ws + off);
    off += up256(split_part_bytes(g.ntiles, g.sk, M));
    // this matrix's share of the 256 workgroups
    int budget = (int)((long long)256 * g.ntiles * g.nS / total);
    budget = budget < 1 ? 1 : budget;
    const size_t per_part = (size_t)M * NDIG * g.spi * 512;
    if (fixed + per_part > 160 * 1024) return CBK_ERR_UNSUPPORTED;
    int pps_max = (int)((160 * 1024 - fixed) / per_part);
    pps_max = pps_max < g.sk ? pps_max : g.sk;
    // Parts per slab: a workgroup runs ceil(items / 16) rounds of one part per wavefront after
    // staging its slab (a 512-column step of M = 8 rows costs about 0.15 rounds of one step)
    float best = 0.f;
    int best_pps = 0;
    for (int pps = 1; pps <= pps_max; ++pps) {
      const int nslab = (g.sk + pps - 1) / pps;
      if (nslab > budget && pps < pps_max) continue;                // (more slabs than workgroups: longer slabs)
      int wps = budget / nslab;
      wps = wps < 1 ? 1 : (wps > g.ntiles ? g.ntiles : wps);
      const int tpw = (g.ntiles + wps - 1) / wps;
      const float c = (float)((tpw * pps + GV_WAVES - 1) / GV_WAVES * g.spi) + 0.15f * (float)M / 8.f * (float)(pps * g.spi);
      if (best_pps == 0 || c < best) { best = c; best_pps = pps; }
    }
    q.g.sp = best_pps;
    q.nslab = (g.sk + best_pps - 1) / best_pps;
    q.wps = budget / q.nslab;
    q.wps = q.wps < 1 ? 1 : (q.wps > g.ntiles ? g.ntiles : q.wps);
    q.tq = g.ntiles / q.wps; q.tr = g.ntiles % q.wps;
    q.inv_wps = q.wps > 1 ? (uint32_t)(((1ull << 32) + q.wps - 1) / q.wps) : 0u;   // exact: workgroup index * wps < 2^32
    q.g.inv_sp = (uint32_t)((65536 + best_pps - 1) / best_pps);
    q.g.dq_t = GV_WAVES / best_pps; q.g.dq_p = GV_WAVES % best_pps;
    const int cols = best_pps * g.spi * 512 < g.m.N ? best_pps * g.spi * 512 : g.m.N;
    xq_cap = xq_cap > M * NDIG * (cols + X_PAD) ? xq_cap : M * NDIG * (cols + X_PAD);
    q.wg0 = wg; wg += q.nslab * q.wps; a.h.wg_end[i] = wg;
    q.th0 = th; th += (g.ntiles * M * 16 + GS_RED_THREADS - 1) / GS_RED_THREADS * GS_RED_THREADS; a.h.th_end[i] = th;
  }
  for (int i = n; i < GV_MAX_BATCH; ++i) { a.h.wg_end[i] = 0x7fffffff; a.h.th_end[i] = 0x7fffffff; }
  a.h.xq_cap = xq_cap; a.h.delta_cap = delta_cap;
  const size_t lds = (size_t)LUT_BYTES + ZERO_BYTES + xq_cap + (size_t)delta_cap * 4;
  if (lds > 160 * 1024) return CBK_ERR_UNSUPPORTED;
  const DMat& m = mats[0].m;
  const int keep = family_of(m.layout) == FAM_DENSE ? 0 : m.keep;
  const bool big = M > 4;
  const int rb = th / GS_RED_THREADS;
  if (m.group != 128) return CBK_ERR_UNSUPPORTED;
  if (m.bits == 4 && keep == 16) return big ? launch_split_cfg<4, 16, 128, 8>(a, lds, wg, rb, st) : launch_split_cfg<4, 16, 128, 4>(a, lds, wg, rb, st);
  if (m.bits == 4 && keep == 0) return big ? launch_split_cfg<4, 0, 128, 8>(a, lds, wg, rb, st) : launch_split_cfg<4, 0, 128, 4>(a, lds, wg, rb, st);
  if (m.bits == 2 && keep == 16) return big ? launch_split_cfg<2, 16, 128, 8>(a, lds, wg, rb, st) : launch_split_cfg<2, 16, 128, 4>(a, lds, wg, rb, st);
  if (m.bits == 2 && keep == 0) return big ? launch_split_cfg<2, 0, 128, 8>(a, lds, wg, rb, st) : launch_split_cfg<2, 0, 128, 4>(a, lds, wg, rb, st);
  return CBK_ERR_UNSUPPORTED;
}

// Distribution over the workgroups, LDS and launch of the matrices of `gb` (spi and sk set).
static int launch_main_batch(GvBatch& gb, hipStream_t st) {
  const int n = gb.h.n, M = gb.h.M;
  int cost = 0, tiles = 0, delta_cap = 0, sk_cap = 1, xq_cap = 0;
  for (int i = 0; i < n; ++i) {
    GvMat& g = gb.mat[i];
    g.cost0 = cost;
    cost += g.ntiles * g.nS;
    gb.h.cost_end[i] = cost;
    tiles += g.ntiles;
    delta_cap = delta_cap > M * (g.m.N / 128 + 4) ? delta_cap : M * (g.m.N / 128 + 4);
    sk_cap = sk_cap > g.sk ? sk_cap : g.sk;
  }
  for (int i = n; i < GV_MAX_BATCH; ++i) gb.h.cost_end[i] = 0x7fffffff;
  const int blocks = gemv_blocks(gb, n, tiles);
  // LDS: selector table, zero row and counters, the deltas, the reduction slots, and the activation
  // digits, which get what the others leave: at least two reduction slots are kept back (up to 24 KB
  // of them where there is room), so that eight rows of 5376 columns (126 KB of digits) are still
  // staged whole.  Rows whose digits do not fit are staged in column slabs: as many whole parts as the
  // budget holds (a part is at most 8 steps = 4096 columns, 12 KB per activation row, so one part of
  // eight rows always fits).
  const size_t slot_bytes = (size_t)sk_cap * M * 16 * 4;
  const size_t fixed = (size_t)LUT_BYTES + ZERO_BYTES + CNT_BYTES + (size_t)delta_cap * 4;
  const size_t x_budget = M == 1 ? (size_t)X_LDS_BUDGET : main_x_budget(M, delta_cap, sk_cap);
  for (int i = 0; i < n; ++i) {
    GvMat& g = gb.mat[i];
    const int N = g.m.N;
    g.sp = g.sk;
    if ((size_t)M * NDIG * (N + X_PAD) > x_budget) {
      g.sp = (int)((x_budget - (size_t)M * NDIG * X_PAD) / ((size_t)M * NDIG * g.spi * 512));
      if (g.sp < 1 || M == 1) return CBK_ERR_UNSUPPORTED;         // (the one-row kernels stage whole rows only)
      const int nsl = (g.sk + g.sp - 1) / g.sp;                   // slabs of equal length, not a short last one
      g.sp = (g.sk + nsl - 1) / nsl;
    }
    const int slab_cols = g.sp >= g.sk ? N : g.sp * g.spi * 512;
    xq_cap = xq_cap > M * NDIG * (slab_cols + X_PAD) ? xq_cap : M * NDIG * (slab_cols + X_PAD);
    if (g.sp > g.sk) g.sp = g.sk;
    // exact for every a the kernel divides (a < cost + nS) when (cost + nS) * nS < 2^32
    g.inv_nS = g.nS > 1 && (uint64_t)(cost + g.nS) * g.nS < (1ull << 32) ? (uint32_t)(((1ull << 32) + g.nS - 1) / g.nS) : 0u;
    g.inv_sp = (uint32_t)((65536 + g.sp - 1) / g.sp);
    g.dq_t = GV_WAVES / g.sp; g.dq_p = GV_WAVES % g.sp;
  }
  gb.h.xq_cap = xq_cap; gb.h.delta_cap = delta_cap;
  // reduction slots: as many as fit what is left, at most 24 KB: a power of two between 2 and 64
  const int slot_floats = sk_cap * M * 16;
  size_t red_room = 160 * 1024 - fixed - (size_t)xq_cap;
  red_room = red_room < 24 * 1024 ? red_room : 24 * 1024;
  int nslot = 64;
  while (nslot > 2 && (size_t)nslot * slot_bytes > red_room) nslot >>= 1;
  gb.h.sk_cap = sk_cap; gb.h.nslot = nslot; gb.h.red_floats = nslot * slot_floats;
  gb.h.cq = cost / blocks; gb.h.cr = cost % blocks;
  const size_t lds = (size_t)LUT_BYTES + ZERO_BYTES + CNT_BYTES + xq_cap + (size_t)delta_cap * 4 +
                     (size_t)gb.h.red_floats * 4;
  if (lds > 160 * 1024) return CBK_ERR_UNSUPPORTED;
  const int bits = gb.mat[0].m.bits;
  if (bits == 6) return launch_mp<6, 16, 128>(gb, lds, blocks, st);   // BLK1632_6: one configuration
  return bits == 2 ? launch_keep<2>(gb, lds, blocks, st) : bits == 3 ? launch_keep<3>(gb, lds, blocks, st)
       : bits == 4 ? launch_keep<4>(gb, lds, blocks, st) : CBK_ERR_UNSUPPORTED;
}

// All matrices share one kernel configuration (checked by the caller) and 1 <= M <= 8 (more than
// four only where gemv_fast_takes says so).
int launch_gemv_fast_batch(int n, const GvCall* calls, int xdt, int M, int ydt, void* workspace, size_t ws_bytes,
                           hipStream_t st) {
  if (n < 1 || n > GV_MAX_BATCH) return CBK_ERR_SHAPE;
  GvBatch gb;
  const int par = calls[0].par ? 1 : 0;
  for (int i = 0; i < n; ++i)
    if ((calls[i].par ? 1 : 0) != par || (calls[i].m.cs_rows == 2) != (par == 1)) return CBK_ERR_UNSUPPORTED;
  M *= par + 1;                                                   // activation rows as the kernel counts them
  if (M > GV_MAX_M) return CBK_ERR_SHAPE;
  gb.h.n = n; gb.h.M = M; gb.h.xdt = xdt; gb.h.ydt = ydt;
  int cost = 0, delta_cap = 0, tiles = 0;
  for (int i = 0; i < n; ++i) {
    const DMat& m = calls[i].m;
    const bool dense = family_of(m.layout) == FAM_DENSE;
    GvMat& g = gb.mat[i];
    g.m = m; g.x = (const uint16_t*)calls[i].x; g.ldx = calls[i].ldx;
    g.order = !dense ? 0 : (m.bits == 2 ? 2 : 1);
    g.par = par;
    g.y = calls[i].y; g.bias = calls[i].bias; g.ldy = calls[i].ldy;
    g.ntiles = (m.K + 15) / 16; g.nS = (m.N / 128 + 3) / 4; g.cost0 = cost;
    g.tile_a = (uint32_t)m.stride * 16u;                          // sixteen rows in either order
    g.lane_mul = m.tiled ? 16u : (uint32_t)m.stride;
    g.sz_mul = m.tiled ? 1u : (uint32_t)m.G;
    g.ush = m.tiled ? 8 : 4; g.csh = m.tiled ? 4 : 0;
    cost += g.ntiles * g.nS;
    tiles += g.ntiles;
    delta_cap = delta_cap > M * (m.N / 128 + 4) ? delta_cap : M * (m.N / 128 + 4);
  }
  const int blocks = gemv_blocks(gb, n, tiles);
  // The parts depend on the matrices of the call only, not on M: they fix the order of every
  // row's partial sums.
  const int spi = launch_spi(cost, blocks);
  int sk_cap = 1;
  for (int i = 0; i < n; ++i) {
    GvMat& g = gb.mat[i];
    row_parts(g.nS, spi, g.spi, g.sk);
    sk_cap = sk_cap > g.sk ? sk_cap : g.sk;
  }
  // Matrices for the column-split kernel (one launch pair for all of them, behind the others),
  // where the configuration has one and the caller has left room for the part sums: rows whose
  // digits do not fit the staging area of the main kernel, and, in launches of at most
  // SPLIT_MAX_TILES tiles, rows whose digits take more than SPLIT_MIN_BYTES of it (eight rows of
  // 5376 columns: every workgroup of the main kernel converts all of them before its first step
  // and is left with four reduction slots; gate,up of that shape 43 us there, 30 + 5 us split).
  // Otherwise the main kernel stages long rows slab by slab.
  const DMat& m0 = gb.mat[0].m;
  if (M > 1 && block_split_capable(m0.bits, family_of(m0.layout) == FAM_DENSE ? 0 : m0.keep, m0.group)) {
    const size_t x_budget = main_x_budget(M, delta_cap, sk_cap);
    auto splits = [&](const GvMat& g) {
      const size_t digits = (size_t)M * NDIG * (g.m.N + X_PAD);
      return digits > x_budget || (digits > SPLIT_MIN_BYTES && tiles <= SPLIT_MAX_TILES);
    };
    GvMat split[GV_MAX_BATCH];
    int ns = 0;
    size_t need = 0;
    for (int i = 0; i < n; ++i) {
      if (splits(gb.mat[i])) {
        split[ns++] = gb.mat[i];
        need += up256(split_part_bytes(gb.mat[i].ntiles, gb.mat[i].sk, M));
      }
    }
    if (ns > 0 && workspace && !((uintptr_t)workspace & 15) && ws_bytes >= need) {
      int na = 0;
      for (int i = 0; i < n; ++i) {
        const GvMat g = gb.mat[i];
        if (!splits(g)) gb.mat[na++] = g;
      }
      gb.h.n = na;
      if (na > 0) {
        const int rc = launch_main_batch(gb, st);
        if (rc != CBK_OK) return rc;
      }
      return launch_split_batch(split, ns, M, xdt, ydt, (uint8_t*)workspace, st);
    }
  }
  return launch_main_batch(gb, st);
}

}  // namespace cbk
