// Measurement aid, not part of any product path: the rate of a register-only MFMA loop, i.e. what the matrix pipes
// of this GPU sustain when nothing else limits them -- with constant operands and with normally distributed ones.
// The second figure is the ceiling a bf16 product can be held against: on random data the chip lowers clock and
// issue rate (switching activity costs power), which no kernel can schedule around.
#include "common.h"

namespace rtp {

typedef __attribute__((ext_vector_type(16))) float probe_f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

// 0: constant operands; 1: about N(0, 1) (a sum of four uniforms), different in every lane and register
__device__ __forceinline__ __bf16 probe_value(unsigned seed, int random_operands) {
  if (!random_operands) return (__bf16)1.0f;
  float s = 0.0f;
  for (int i = 0; i < 4; ++i) s += (float)(probe_hash(seed * 4u + i) & 0xffff) / 65536.0f - 0.5f;
  return (__bf16)(s * 1.7f);
}

// 4 wavefronts per workgroup; per iteration a wavefront issues 32 v_mfma_f32_32x32x16_bf16 on 4 independent
// accumulators, cycling through 8 A and 8 B fragments that never leave their registers.
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* sink, int iters, int random_operands) {
  probe_bf16x8 a[8], b[8];
  for (int j = 0; j < 8; ++j)
    for (int e = 0; e < 8; ++e) {
      const unsigned id = (blockIdx.x * 256 + threadIdx.x) * 64 + j * 8 + e;
      a[j][e] = probe_value(id, random_operands);
      b[j][e] = probe_value(id + 7777777u, random_operands);
    }
  probe_f32x16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(j + i) & 7], b[j], acc[i], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 4; ++i) s += acc[i][0];
  if (s == 123.456f) sink[0] = s;  // keeps the loop alive; never true for these operands
}

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_probe_mfma_rate(void* stream, int random_operands, int iters, double* tflops) {
  RTP_REQUIRE(tflops && iters >= 1 && iters <= (1 << 20), "rtp_probe_mfma_rate: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  float* sink = nullptr;
  RTP_HIP_TRY(hipMalloc(&sink, sizeof(float)));
  hipEvent_t e0, e1;
  RTP_HIP_TRY(hipEventCreate(&e0));
  RTP_HIP_TRY(hipEventCreate(&e1));
  const int wgs = 512;  // two workgroups per CU: 2 wavefronts per SIMD keep the pipe fed across dependent MFMAs
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(wgs), dim3(256), 0, st, sink, iters / 10 + 1, random_operands);  // warm-up
  RTP_HIP_TRY(hipEventRecord(e0, st));
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(wgs), dim3(256), 0, st, sink, iters, random_operands);
  RTP_HIP_TRY(hipEventRecord(e1, st));
  RTP_HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.0f;
  RTP_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  RTP_HIP_TRY(hipEventDestroy(e0));
  RTP_HIP_TRY(hipEventDestroy(e1));
  RTP_HIP_TRY(hipFree(sink));
  *tflops = (double)wgs * 4.0 * iters * 32.0 * 32768.0 / (ms * 1e-3) / 1e12;
  return RTP_OK;
}
