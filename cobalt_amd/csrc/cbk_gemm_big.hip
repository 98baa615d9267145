// Prefill GEMM for M > 128:  Y[M, K] = X[M, N] . W_hat[K, N]^T on the gfx950 matrix cores.
//
// Workgroup tile 256 tokens x 256 weight rows, 64 input columns per stage, four wavefronts
// each owning a 128 x 128 sub-tile (4 x 4 blocks of v_mfma_f32_32x32x16_f16, 256 accumulator
// registers), one wavefront per SIMD.  Both operands are double-buffered in LDS (147 KB):
// while the matrix cores work on stage s, the same wavefronts dequantise the weights of
// stage s + 1 into the other buffer and copy the activation tile there.
//
// Operands.  The activation side is X' = fp16(x * col_scale), written once per call into the
// caller's workspace by a small elementwise kernel (bf16 inputs are widened exactly; the
// product is rounded once to fp16, magnitudes above 65504 saturate).  The weight side is
// fp16((q - zero) * scale) for a kept column and exactly 0 for a pruned one, so
// Y = sum_j X'[m,j] * W'[k,j] carries two roundings of relative size 2^-12.  Feeding bf16
// operands instead would round to 2^-9, which alone exceeds the 1e-3 relative-Frobenius
// budget of this layer; the f16 and bf16 MFMA rates are identical.
//
// Weight decode.  Each of the 256 threads owns one weight row of the tile and decodes its
// 64 columns of the stage.  For 4-bit codes with 16 of 32 kept, and for the dense 4-bit
// layout, this is the byte-permute decoder of the decode kernel (selector table in LDS)
// followed by two packed-half operations per column pair; other configurations go through
// the generic 32-column reader.
//
// Workgroups are ordered so that those running at the same time on one XCD (blockIdx % 8)
// share their token tile, which then stays in that XCD's L2.
//
// Reference semantics: cbk::gemm_tile (src/cobaltkernel/csrc/cobalt_gemm.cuh:243-609).
#include <atomic>
#include <type_traits>
#include "cbk_device.h"

namespace cbk {

constexpr int GB_T = 256;       // tokens per workgroup tile
constexpr int GB_R = 256;       // weight rows per workgroup tile
constexpr int GB_K = 64;        // input columns per stage
constexpr int GB_P = GB_K + 8;  // LDS row pitch in halfs (144 B): conflict-free 16-byte reads
constexpr int GB_LUT = 256 * 8 * 8;   // selector table, 8 lane-private copies of 256 x 8 B

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

__device__ inline uint2 gb_selectors(uint32_t mb) {
  uint32_t lo = 0, hi = 0, r = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const uint32_t idx = (r >> 1) + 4u * (r & 1u);
    const bool kp = (mb >> p) & 1u;
    const uint32_t sel = kp ? idx : 0x0Cu;
    if (p < 4) lo |= sel << (8 * p); else hi |= sel << (8 * (p - 4));
    r += kp ? 1u : 0u;
  }
  return make_uint2(lo, hi);
}

// ---- X' = fp16(x * col_scale), [Mpad, N] row-major, rows M..Mpad-1 zero
__global__ __launch_bounds__(256) void gemm_prep_kernel(const uint16_t* x, int64_t ldx, const uint16_t* cs, int xdt,
                                                        int M, int Mpad, int N, uint16_t* out) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;     // one thread = 8 columns
  const int n8 = N >> 3;
  if (id >= (int64_t)Mpad * n8) return;
  const int row = (int)(id / n8), c8 = (int)(id % n8);
  if (row >= M) { *(uint4*)(out + (size_t)row * N + c8 * 8) = make_uint4(0, 0, 0, 0); return; }
  const uint4 v = *(const uint4*)(x + (size_t)row * ldx + c8 * 8);
  uint4 c = make_uint4(0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u);
  if (cs) c = *(const uint4*)(cs + c8 * 8);
  const uint32_t xw[4] = {v.x, v.y, v.z, v.w}, cw[4] = {c.x, c.y, c.z, c.w};
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float a0, a1;
    if (xdt == CBK_F16) { a0 = h2f((uint16_t)(xw[e] & 0xffffu)); a1 = h2f((uint16_t)(xw[e] >> 16)); }
    else { a0 = bf2f((uint16_t)(xw[e] & 0xffffu)); a1 = bf2f((uint16_t)(xw[e] >> 16)); }
    a0 *= h2f((uint16_t)(cw[e] & 0xffffu)); a1 *= h2f((uint16_t)(cw[e] >> 16));
    a0 = fminf(fmaxf(a0, -65504.f), 65504.f); a1 = fminf(fmaxf(a1, -65504.f), 65504.f);
    o[e] = (uint32_t)f2h(a0) | ((uint32_t)f2h(a1) << 16);
  }
  *(uint4*)(out + (size_t)row * N + c8 * 8) = make_uint4(o[0], o[1], o[2], o[3]);
}

struct GbArgs {
  DMat m;
  const uint16_t* xp;      // X' fp16 [M, N]
  int M;
  void* y;
  int ydt;
  int64_t ldy;
  const void* bias;
  int tiles_t, tiles_r;
};

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

// FAST: 0 generic reader, 1 bitmap 16-of-32 4-bit, 2 dense 4-bit  (group 128 in both fast modes)
template <int FAST>
__global__ __launch_bounds__(256) void gemm_big_kernel(GbArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  _Float16* Xs = (_Float16*)smem;                                 // [2][GB_T][GB_P]
  _Float16* Ws = Xs + 2 * GB_T * GB_P;                            // [2][GB_R][GB_P]
  uint2* lut = (uint2*)(Ws + 2 * GB_R * GB_P);                    // [256][8]
  const DMat& m = a.m;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wt = wave >> 1, wr = wave & 1;
  // XCD-aware order: blockIdx % 8 picks the XCD; give each XCD whole token tiles
  const int nb = a.tiles_t * a.tiles_r;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int per = (nb + 7) >> 3;
  const int lin = xcd * per + idx;                                 // token-tile-major linear id
  if (lin >= nb) return;
  const int tt = lin / a.tiles_r, tr = lin % a.tiles_r;
  const int t0 = tt * GB_T, r0 = tr * GB_R;
  const int N = m.N, nst = N / GB_K;

  if (FAST == 1) {
    const uint2 e = gb_selectors((uint32_t)tid);
#pragma unroll
    for (int j = 0; j < 8; ++j) lut[tid * 8 + j] = e;
  }
  const uint32_t l8 = lane & 7;

  v16f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // this thread's weight row
  const int wrow = r0 + tid;
  const bool wok = wrow < m.K;
  const int wrc = wok ? wrow : m.K - 1;
  const RowView rv = row_view(m, wrc);
  const size_t meta0 = meta_index(m, wrc, 0), meta_step = m.tiled ? 16 : 1;
  // activation rows this thread copies: 8 x 16 B per stage, rows tid/8 + 32 i (X' is padded
  // to whole token tiles, so no bounds checks)
  const uint16_t* xsrc = a.xp + (size_t)(t0 + (tid >> 3)) * N + (tid & 7) * 8;
  const size_t xstep = (size_t)32 * N;
  const uint32_t xdst = (uint32_t)((tid >> 3) * GB_P + (tid & 7) * 8);

  uint4 xr0, xr1, xr2, xr3, xr4, xr5, xr6, xr7;                   // named: an array here ends up on the stack
  struct WReg { uint32_t m[2]; uint32_t c[8]; uint32_t z; float s; };
  WReg w0, w1;                                                    // stages of even / odd parity

  auto load_x = [&](int s) {
    const uint16_t* p = xsrc + s * GB_K;
    xr0 = *(const uint4*)(p);             xr1 = *(const uint4*)(p + xstep);
    xr2 = *(const uint4*)(p + 2 * xstep); xr3 = *(const uint4*)(p + 3 * xstep);
    xr4 = *(const uint4*)(p + 4 * xstep); xr5 = *(const uint4*)(p + 5 * xstep);
    xr6 = *(const uint4*)(p + 6 * xstep); xr7 = *(const uint4*)(p + 7 * xstep);
  };
  auto load_w = [&](int s, WReg& w) {
    const int c0 = s * GB_K;
    if (FAST == 1) {
      // mask: 8 bytes at byte c0/8 of the row; codes: 16 bytes at code plane + c0/4
      const uint32_t md = (uint32_t)c0 >> 5;
      w.m[0] = rv.dword(md); w.m[1] = rv.dword(md + 1);
      const uint4 v = *(const uint4*)rv.unit((m.code_off >> 4) + ((uint32_t)c0 >> 6));
      w.c[0] = v.x; w.c[1] = v.y; w.c[2] = v.z; w.c[3] = v.w;
    } else if (FAST == 2) {
      const uint4 v0 = *(const uint4*)rv.unit((uint32_t)c0 >> 5), v1 = *(const uint4*)rv.unit(((uint32_t)c0 >> 5) + 1);
      w.c[0] = v0.x; w.c[1] = v0.y; w.c[2] = v0.z; w.c[3] = v0.w; w.c[4] = v1.x; w.c[5] = v1.y; w.c[6] = v1.z; w.c[7] = v1.w;
    }
    if (FAST != 0) {
      const size_t mi = meta0 + (size_t)(c0 >> 7) * meta_step;
      w.z = m.zero[mi];
      w.s = h2f(m.scale[mi]);
    }
  };

  // decode the staged weights of stage s into Ws[buf], quarter qq (16 columns) at a time
  // selectors of the two mask bytes of quarter qq (bitmap layout only)
  auto fetch_sel = [&](const WReg& w, int qq, uint2 (&sel)[2]) {
    if (FAST != 1) return;
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
      const int jb8 = qq * 2 + hb;
      const uint32_t mb = (w.m[jb8 >> 2] >> (8 * (jb8 & 3))) & 0xFFu;
      sel[hb] = lut[mb * 8 + l8];
    }
  };
  auto store_w_quarter = [&](int s, const WReg& w, int buf, int qq, const uint2 (&selq)[2]) {
    _Float16* dst = Ws + (size_t)buf * GB_R * GB_P + tid * GB_P + qq * 16;
    if (FAST == 0) {
      if (qq & 1) return;                                         // the generic reader works on 32 columns
      uint32_t packed[16];
      if (wok) {
        int q[32];
        const int t = (s * GB_K >> 5) + (qq >> 1);
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
    const _Float16 sh = (_Float16)(wok ? w.s : 0.f);
    const h2_t s2 = {sh, sh};
    const uint32_t nz = 0x80808080u - w.z * 0x01010101u;
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {                              // two mask bytes = 16 columns
      const int jb8 = qq * 2 + hb;                                // mask byte of the stage, 0..7
      uint32_t b0, b1;
      if (FAST == 1) {
        const uint32_t mw = w.m[jb8 >> 2];
        const int jj = jb8 & 3;
        const uint32_t r = jj == 0 ? 0u : (uint32_t)__builtin_popcount(mw & ((1u << (8 * jj)) - 1u));
        const uint64_t st = ((uint64_t)w.c[2 * (jb8 >> 2) + 1] << 32) | w.c[2 * (jb8 >> 2)];
        const uint32_t cw = (uint32_t)(st >> ((r * 4u) & 63u));
        const uint32_t p0 = ((cw & 0x0F0F0F0Fu) + nz) ^ 0x80808080u;
        const uint32_t p1 = (((cw >> 4) & 0x0F0F0F0Fu) + nz) ^ 0x80808080u;
        b0 = __builtin_amdgcn_perm(p1, p0, selq[hb].x);
        b1 = __builtin_amdgcn_perm(p1, p0, selq[hb].y);
      } else {
        const uint32_t cw = w.c[jb8];
        const uint32_t p0 = ((cw & 0x0F0F0F0Fu) + nz) ^ 0x80808080u;          // even columns
        const uint32_t p1 = (((cw >> 4) & 0x0F0F0F0Fu) + nz) ^ 0x80808080u;   // odd columns
        b0 = __builtin_amdgcn_perm(p1, p0, 0x05010400u);
        b1 = __builtin_amdgcn_perm(p1, p0, 0x07030602u);
      }
      ((uint4*)dst)[hb] = bytes_to_halfs(b0, b1, s2);
    }
  };
  auto store_x = [&](int buf) {
    _Float16* base = Xs + (size_t)buf * GB_T * GB_P + xdst;
    *(uint4*)(base) = xr0;                 *(uint4*)(base + 32 * GB_P) = xr1;
    *(uint4*)(base + 64 * GB_P) = xr2;     *(uint4*)(base + 96 * GB_P) = xr3;
    *(uint4*)(base + 128 * GB_P) = xr4;    *(uint4*)(base + 160 * GB_P) = xr5;
    *(uint4*)(base + 192 * GB_P) = xr6;    *(uint4*)(base + 224 * GB_P) = xr7;
  };

  // ---- prologue: stage 0 into buffer 0; stage 1 into registers (X in xr, W in w1)
  load_x(0); load_w(0, w0);
  __syncthreads();                                                // selector table visible
  store_x(0);
#pragma unroll
  for (int qq = 0; qq < 4; ++qq) {
    uint2 sel[2];
    fetch_sel(w0, qq, sel);
    store_w_quarter(0, w0, 0, qq, sel);
  }
  load_w(1, w1); load_x(1);
  uint2 selq[2];                                                  // selectors of the next quarter to decode
  fetch_sel(w1, 0, selq);
  __syncthreads();

  // One stage: matrix-core work on buffer s % 2.  With MORE, the registers holding stage
  // s + 1 are written to the other buffer (X as is, W decoded a quarter at a time between the
  // MFMAs) and stage s + 2 (clamped to the last) is fetched into the registers just freed,
  // so every global load has a whole stage in which to land.  wd: registers of stage s + 1,
  // wl: registers that receive stage s + 2.  No branches inside.
  auto stage = [&](int s, auto more_tag, const WReg& wd, WReg& wl) {
    constexpr bool MORE = decltype(more_tag)::value;
    const int buf = s & 1;
    const _Float16* xb = Xs + (size_t)buf * GB_T * GB_P + (128 * wt + (lane & 31)) * GB_P + 8 * (lane >> 5);
    const _Float16* wb = Ws + (size_t)buf * GB_R * GB_P + (128 * wr + (lane & 31)) * GB_P + 8 * (lane >> 5);
    v8h af[2][4], bf[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) af[0][i] = *(const v8h*)(xb + 32 * i * GB_P);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[0][j] = *(const v8h*)(wb + 32 * j * GB_P);
    // the X registers of stage s + 1 go to LDS two per phase; the loads of stage s + 2 below
    // land in fresh registers (the old ones stay live until their store)
    const uint4 xo0 = xr0, xo1 = xr1, xo2 = xr2, xo3 = xr3, xo4 = xr4, xo5 = xr5, xo6 = xr6, xo7 = xr7;
    _Float16* xw = Xs + (size_t)(buf ^ 1) * GB_T * GB_P + xdst;
    if (MORE) {
      const int s2 = s + 2 < nst ? s + 2 : nst - 1;
      load_w(s2, wl);                                             // first: its data is wanted first
      load_x(s2);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < GB_K / 16; ++kk) {
      const int c = kk & 1, n = c ^ 1;
      if (kk + 1 < GB_K / 16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) af[n][i] = *(const v8h*)(xb + 32 * i * GB_P + 16 * (kk + 1));
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[n][j] = *(const v8h*)(wb + 32 * j * GB_P + 16 * (kk + 1));
      }
      // selectors one quarter ahead, so that their LDS latency is never waited for
      uint2 seln[2];
      if (kk + 1 < GB_K / 16) fetch_sel(wd, kk + 1, seln); else fetch_sel(wl, 0, seln);
      if (MORE) {
        if (kk == 0) { *(uint4*)(xw) = xo0;              *(uint4*)(xw + 32 * GB_P) = xo1; }
        if (kk == 1) { *(uint4*)(xw + 64 * GB_P) = xo2;  *(uint4*)(xw + 96 * GB_P) = xo3; }
        if (kk == 2) { *(uint4*)(xw + 128 * GB_P) = xo4; *(uint4*)(xw + 160 * GB_P) = xo5; }
        if (kk == 3) { *(uint4*)(xw + 192 * GB_P) = xo6; *(uint4*)(xw + 224 * GB_P) = xo7; }
        store_w_quarter(s + 1, wd, buf ^ 1, kk, selq);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[c][i], bf[c][j], acc[i][j], 0, 0, 0);
      selq[0] = seln[0]; selq[1] = seln[1];
#pragma unroll
      for (int g = 0; g < 16; ++g) {                              // one MFMA, then a slice of the decode
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  };
  // N is a multiple of 128, so the number of stages is even.  The last stage also decodes
  // (the clamped, already consumed) registers into the idle buffer: one loop body, no tail.
  for (int s = 0; s < nst; s += 2) {
    stage(s, std::true_type{}, w1, w0);
    stage(s + 1, std::true_type{}, w0, w1);
  }

  // ---- epilogue: D[i][j] with j = lane%32 (weight row), i = 8*(r/4) + 4*(lane/32) + r%4 (token)
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int k = r0 + 128 * wr + 32 * j + (lane & 31);
    if (k >= m.K) continue;
    float bv = 0.f;
    if (a.bias) bv = (a.ydt == CBK_F32) ? ((const float*)a.bias)[k]
                   : (a.ydt == CBK_F16) ? h2f(((const uint16_t*)a.bias)[k]) : bf2f(((const uint16_t*)a.bias)[k]);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int tok = t0 + 128 * wt + 32 * i + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (tok >= a.M) continue;
        const float v = acc[i][j][r] + bv;
        const size_t o = (size_t)tok * a.ldy + k;
        if (a.ydt == CBK_F32) ((float*)a.y)[o] = v;
        else if (a.ydt == CBK_F16) ((uint16_t*)a.y)[o] = f2h(v);
        else ((uint16_t*)a.y)[o] = f2bf(v);
      }
  }
}

size_t gemm_big_workspace(const DMat& m, int M) {
  const size_t mpad = (size_t)(M + GB_T - 1) / GB_T * GB_T;
  return (mpad * m.N * 2 + 255) & ~(size_t)255;
}

template <int FAST>
static int launch_big(const GbArgs& a, int blocks, hipStream_t st) {
  auto kern = gemm_big_kernel<FAST>;
  static std::atomic<int> configured{0};
  const size_t lds = (size_t)2 * (GB_T + GB_R) * GB_P * 2 + GB_LUT;
  if (!configured.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
      return CBK_ERR_HIP;
    configured.store(1, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, st, a);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

int launch_gemm_big(const DMat& m, const void* x, int xdt, int M, int64_t ldx, void* y, int ydt, int64_t ldy,
                    const void* bias, void* ws, size_t ws_bytes, hipStream_t st) {
  if (family_of(m.layout) == FAM_SPARSE) return CBK_ERR_UNSUPPORTED;
  if (m.cs_rows > 1) return CBK_ERR_UNSUPPORTED;
  if (!ws || ws_bytes < gemm_big_workspace(m, M)) return CBK_ERR_WORKSPACE;
  if ((uintptr_t)ws & 255) return CBK_ERR_ALIGN;
  const int Mpad = (M + GB_T - 1) / GB_T * GB_T;
  const int64_t items = (int64_t)Mpad * (m.N / 8);
  hipLaunchKernelGGL(gemm_prep_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st,
                     (const uint16_t*)x, ldx, m.cs, xdt, M, Mpad, m.N, (uint16_t*)ws);
  GbArgs a;
  a.m = m; a.xp = (const uint16_t*)ws; a.M = M; a.y = y; a.ydt = ydt; a.ldy = ldy; a.bias = bias;
  a.tiles_t = (M + GB_T - 1) / GB_T; a.tiles_r = (m.K + GB_R - 1) / GB_R;
  const int nb = a.tiles_t * a.tiles_r;
  const int blocks = ((nb + 7) / 8) * 8;
  const bool le128 = (m.flags & CBK_FLAG_ZERO_LE_128) != 0;
  const int fam = family_of(m.layout);
  if (le128 && fam == FAM_BLK && m.bits == 4 && m.keep == 16 && m.group == 128) return launch_big<1>(a, blocks, st);
  if (le128 && fam == FAM_DENSE && m.bits == 4 && m.group == 128) return launch_big<2>(a, blocks, st);
  return launch_big<0>(a, blocks, st);
}

}  // namespace cbk
