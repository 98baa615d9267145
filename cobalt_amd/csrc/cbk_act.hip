// Gated-MLP epilogue for a gate/up matrix whose rows 2i (gate) and 2i+1 (up) belong together:
//   y[m, i] = act(t[m, 2i]) * t[m, 2i+1],  act = tanh-GELU or SiLU,
// evaluated in float32 and rounded once to the output type.
//
// Reference semantics: EPI_GEGLU_BF16 / EPI_SWIGLU_BF16 of cbk::gemm_tile
// (src/cobaltkernel/csrc/cobalt_gemm.cuh:30-33, :216-220, :586-592).
#include "cbk_device.h"

namespace cbk {

__device__ inline float act_gelu_tanh(float x) {
  const float k = 0.7978845608028654f;                              // sqrt(2 / pi)
  return 0.5f * x * (1.f + tanhf(k * (x + 0.044715f * x * x * x)));
}
__device__ inline float act_silu(float x) { return x / (1.f + __expf(-x)); }

// One thread: eight outputs of one activation row (sixteen consecutive elements of t).
// eight consecutive elements from a 16-byte aligned position
template <int TDT>
__device__ inline void load8(const void* t, size_t at, float (&o)[8]) {
  if (TDT == CBK_F32) {
    const float4* p = (const float4*)((const float*)t + at);
    const float4 a = p[0], b = p[1];
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  } else {
    const uint4 q = *(const uint4*)((const uint16_t*)t + at);
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint16_t lo = (uint16_t)(w[c] & 0xffffu), hi = (uint16_t)(w[c] >> 16);
      o[2 * c] = TDT == CBK_F16 ? h2f(lo) : bf2f(lo);
      o[2 * c + 1] = TDT == CBK_F16 ? h2f(hi) : bf2f(hi);
    }
  }
}

// HALVES: t holds the gate outputs in columns [0, K2) and the up outputs in [K2, 2 K2) instead of
// interleaving them (v[2e], v[2e+1] stay gate, up of output e either way).
template <int TDT, int YDT, int ACT, bool HALVES>
__global__ __launch_bounds__(256) void act_mul_kernel(const void* __restrict__ t, int64_t ldt, void* __restrict__ y,
                                                      int64_t ldy, int M, int K2, const void* __restrict__ bias) {
  const int per_row = (K2 + 7) >> 3;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)M * per_row) return;
  const int m = (int)(id / per_row), i0 = (int)(id % per_row) * 8;
  const size_t tb = (size_t)m * ldt + 2 * (size_t)i0, yb = (size_t)m * ldy + i0;
  float v[16];
  const bool whole = i0 + 8 <= K2;
  constexpr int TSZ = TDT == CBK_F32 ? 4 : 2, YSZ = YDT == CBK_F32 ? 4 : 2;
  if (HALVES) {
    const size_t gb = (size_t)m * ldt + i0, ub = gb + K2;
    if (whole && ((((uintptr_t)t + gb * TSZ) | ((uintptr_t)t + ub * TSZ)) & 15) == 0) {
      float g8[8], u8[8];
      load8<TDT>(t, gb, g8);
      load8<TDT>(t, ub, u8);
#pragma unroll
      for (int e = 0; e < 8; ++e) { v[2 * e] = g8[e]; v[2 * e + 1] = u8[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bool in = i0 + e < K2;
        v[2 * e] = in ? load_act<TDT>(t, gb + e) : 0.f;
        v[2 * e + 1] = in ? load_act<TDT>(t, ub + e) : 0.f;
      }
    }
  } else if (whole && ((((uintptr_t)t + tb * TSZ) & 15) == 0)) {
    if (TDT == CBK_F32) {
      const float4* p = (const float4*)((const float*)t + tb);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float4 q = p[e];
        v[4 * e] = q.x; v[4 * e + 1] = q.y; v[4 * e + 2] = q.z; v[4 * e + 3] = q.w;
      }
    } else {
      const uint4* p = (const uint4*)((const uint16_t*)t + tb);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const uint4 q = p[e];
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint16_t lo = (uint16_t)(w[c] & 0xffffu), hi = (uint16_t)(w[c] >> 16);
          v[8 * e + 2 * c] = TDT == CBK_F16 ? h2f(lo) : bf2f(lo);
          v[8 * e + 2 * c + 1] = TDT == CBK_F16 ? h2f(hi) : bf2f(hi);
        }
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = (i0 + (e >> 1) < K2) ? load_act<TDT>(t, tb + e) : 0.f;
  }
  if (bias) {                                                       // K entries of the output type
#pragma unroll
    for (int e = 0; e < 16; ++e)
      if (i0 + (e >> 1) < K2) v[e] += load_act<YDT>(bias, 2 * (size_t)i0 + e);
  }
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (ACT == CBK_ACT_GELU_TANH ? act_gelu_tanh(v[2 * e]) : act_silu(v[2 * e])) * v[2 * e + 1];
  if (whole && ((((uintptr_t)y + yb * YSZ) & 15) == 0)) {
    if (YDT == CBK_F32) {
      float4* p = (float4*)((float*)y + yb);
      p[0] = make_float4(o[0], o[1], o[2], o[3]);
      p[1] = make_float4(o[4], o[5], o[6], o[7]);
    } else {
      uint32_t w[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint16_t lo = YDT == CBK_F16 ? f2h(o[2 * c]) : f2bf(o[2 * c]);
        const uint16_t hi = YDT == CBK_F16 ? f2h(o[2 * c + 1]) : f2bf(o[2 * c + 1]);
        w[c] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
      *(uint4*)((uint16_t*)y + yb) = make_uint4(w[0], w[1], w[2], w[3]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (i0 + e < K2) store_out<YDT>(y, yb + e, o[e]);
  }
}

template <int TDT, int YDT, bool HALVES>
static int launch_act3(const void* t, int64_t ldt, void* y, int64_t ldy, int M, int K2, int act, const void* bias,
                       hipStream_t st) {
  const int64_t n = (int64_t)M * ((K2 + 7) >> 3);
  const dim3 grid((unsigned)((n + 255) / 256)), blk(256);
  if (act == CBK_ACT_GELU_TANH)
    hipLaunchKernelGGL((act_mul_kernel<TDT, YDT, CBK_ACT_GELU_TANH, HALVES>), grid, blk, 0, st, t, ldt, y, ldy, M, K2, bias);
  else
    hipLaunchKernelGGL((act_mul_kernel<TDT, YDT, CBK_ACT_SILU, HALVES>), grid, blk, 0, st, t, ldt, y, ldy, M, K2, bias);
  return hipGetLastError() == hipSuccess ? CBK_OK : CBK_ERR_HIP;
}

template <int TDT, int YDT>
static int launch_act2(const void* t, int64_t ldt, void* y, int64_t ldy, int M, int K2, int act, const void* bias,
                       hipStream_t st, bool halves) {
  return halves ? launch_act3<TDT, YDT, true>(t, ldt, y, ldy, M, K2, act, bias, st)
                : launch_act3<TDT, YDT, false>(t, ldt, y, ldy, M, K2, act, bias, st);
}

template <int TDT>
static int launch_act1(const void* t, int64_t ldt, void* y, int ydt, int64_t ldy, int M, int K2, int act,
                       const void* bias, hipStream_t st, bool halves) {
  if (ydt == CBK_F32) return launch_act2<TDT, CBK_F32>(t, ldt, y, ldy, M, K2, act, bias, st, halves);
  if (ydt == CBK_F16) return launch_act2<TDT, CBK_F16>(t, ldt, y, ldy, M, K2, act, bias, st, halves);
  if (ydt == CBK_BF16T) return launch_act2<TDT, CBK_BF16T>(t, ldt, y, ldy, M, K2, act, bias, st, halves);
  return CBK_ERR_DTYPE;
}

int launch_act_mul(const void* t, int tdt, int64_t ldt, void* y, int ydt, int64_t ldy, int M, int K2, int act,
                   const void* bias, hipStream_t st, bool halves) {
  if (act != CBK_ACT_GELU_TANH && act != CBK_ACT_SILU) return CBK_ERR_UNSUPPORTED;
  if (M <= 0 || K2 <= 0) return CBK_OK;
  if (tdt == CBK_F32) return launch_act1<CBK_F32>(t, ldt, y, ydt, ldy, M, K2, act, bias, st, halves);
  if (tdt == CBK_F16) return launch_act1<CBK_F16>(t, ldt, y, ydt, ldy, M, K2, act, bias, st, halves);
  if (tdt == CBK_BF16T) return launch_act1<CBK_BF16T>(t, ldt, y, ydt, ldy, M, K2, act, bias, st, halves);
  return CBK_ERR_DTYPE;
}

}  // namespace cbk
