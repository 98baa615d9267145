// Measurement helpers for bench.py, built into their own small library (libcbk_bench.so): what
// this GPU reaches on (a) back-to-back dense f16 MFMAs and (b) a plain streaming read, so that
// a kernel's throughput can be put beside a measured ceiling as well as the published one.
// In the spirit of the reference's own peak probes (src/cobaltkernel/csrc/test_gemm.cu:115-149
// for the matrix pipe, bench_env/bw.cu for memory reads).  Not part of the layer's C ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// One wavefront per SIMD, 16 independent 32x32x16 accumulators: nothing but the matrix pipe.
__global__ __launch_bounds__(256) void bench_mfma_kernel(float* sink, int iters) {
  v16f acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  v8h a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) { a[e] = (_Float16)(threadIdx.x * 0.001f + e); b[e] = (_Float16)(e * 0.5f); }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[i][e];
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// Grid-stride read of 16 bytes per lane, eight loads in flight per lane; the xor keeps the loads.
__global__ __launch_bounds__(256) void bench_read_kernel(const uint4* __restrict__ p, size_t n16, uint32_t* sink) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  uint32_t x = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = p[i + k * stride];
#pragma unroll
    for (int k = 0; k < 8; ++k) x ^= v[k].x ^ v[k].y ^ v[k].z ^ v[k].w;
  }
  for (; i < n16; i += stride) {
    const uint4 a = p[i];
    x ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (x == 0x9e3779b9u) sink[0] = x;                                // practically never: the loads cannot be dropped
}

extern "C" {

// flops of one call: blocks * 4 wavefronts * iters * 16 MFMAs * 2 * 32 * 32 * 16
int cbk_bench_mfma_f16(int blocks, int iters, void* sink /* blocks * 256 floats */, void* stream) {
  if (blocks < 1 || iters < 1 || !sink) return -1;
  hipLaunchKernelGGL(bench_mfma_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (float*)sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

int cbk_bench_read(const void* p, size_t bytes, int blocks, void* sink /* 4 bytes */, void* stream) {
  if (!p || !sink || blocks < 1 || ((uintptr_t)p & 15)) return -1;
  hipLaunchKernelGGL(bench_read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4*)p, bytes / 16,
                     (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

}  // extern "C"
