// Shared helpers for the gfx950 kernels behind the C ABI in include/rtp_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "rtp_hip.h"

namespace rtp {

// Thread-local message behind rtp_last_error().
char* error_buffer();

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

#define RTP_HIP_TRY(expr)                                                                  \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess)                                                                  \
      return ::rtp::fail(RTP_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                         __FILE__, __LINE__);                                              \
  } while (0)

#define RTP_REQUIRE(cond, ...)                              \
  do {                                                      \
    if (!(cond)) return ::rtp::fail(RTP_ERR_ARG, __VA_ARGS__); \
  } while (0)

// A launch error is reported by hipGetLastError right after the <<<>>>.
#define RTP_LAUNCH_CHECK() RTP_HIP_TRY(hipGetLastError())

typedef __bf16 bf16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) {
  return (bf16_t)v;  // round to nearest even
}

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Streaming accesses: data that is touched once per step (home shards read by the rotation copy, optimiser
// state) is loaded and stored non-temporally so that it does not push the matrix-product operands out of the
// L2 and the memory-side cache.
typedef unsigned int nt_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int nt_u32x2 __attribute__((ext_vector_type(2)));
typedef float nt_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 nt_load(const uint4* p) {
  const nt_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 nt_load(const uint2* p) {
  const nt_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x2*>(p));
  return make_uint2(v.x, v.y);
}
__device__ __forceinline__ float4 nt_load(const float4* p) {
  const nt_f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const nt_f32x4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}

// Clip + SGD on one element: g is the gradient as the output dtype holds it.  Two roundings (product, then
// difference), no fused multiply-add: the arithmetic of sgd_kernel in optim.hip.
template <typename T>
__device__ __forceinline__ float sgd_update(float w, float v, float lr, float clip) {
  float g = to_f32(from_f32<T>(v));
  if (clip > 0.0f) g = fminf(fmaxf(g, -clip), clip);
  {
#pragma clang fp contract(off)
    const float step = lr * g;
    return w - step;
  }
}

__device__ __forceinline__ void nt_store(float4 a, float4* p) {
  const nt_f32x4 v = {a.x, a.y, a.z, a.w};
  __builtin_nontemporal_store(v, reinterpret_cast<nt_f32x4*>(p));
}
__device__ __forceinline__ void nt_store(uint2 a, uint2* p) {
  const nt_u32x2 v = {a.x, a.y};
  __builtin_nontemporal_store(v, reinterpret_cast<nt_u32x2*>(p));
}
__device__ __forceinline__ void nt_store(uint4 a, uint4* p) {
  const nt_u32x4 v = {a.x, a.y, a.z, a.w};
  __builtin_nontemporal_store(v, reinterpret_cast<nt_u32x4*>(p));
}

// Resolves, for the current device, the address of the scratch buffer built into the library for
// rtp_gate_wgrad_static (gate.hip).  Part of rtp_device_check.
int gate_static_setup();

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Reads one word of every 64-byte line of a kernel's BYTES bytes of arguments (and of the launch dimensions that
// follow them) in one batch, first thing in the kernel.  The scalar cache is cold at kernel start and the compiler
// fetches arguments where they are first used: a kernel that needs them at three places pays three trips to
// memory in a row, a microsecond in a ten-microsecond kernel.  After this every later fetch hits the cache.
template <size_t BYTES>
__device__ __forceinline__ void touch_kernel_arguments() {
  constexpr int LINES = (int)(BYTES / 64) + 1;
  static_assert(LINES <= 10, "at most 640 bytes of kernel arguments");
  typedef const __attribute__((address_space(4))) int* kernarg_t;
  kernarg_t ka = (kernarg_t)__builtin_amdgcn_kernarg_segment_ptr();
  const int w0 = ka[0], w1 = ka[LINES > 1 ? 16 : 0], w2 = ka[LINES > 2 ? 32 : 0], w3 = ka[LINES > 3 ? 48 : 0];
  const int w4 = ka[LINES > 4 ? 64 : 0], w5 = ka[LINES > 5 ? 80 : 0], w6 = ka[LINES > 6 ? 96 : 0];
  const int w7 = ka[LINES > 7 ? 112 : 0], w8 = ka[LINES > 8 ? 128 : 0], w9 = ka[LINES > 9 ? 144 : 0];
  asm volatile("" ::"s"(w0), "s"(w1), "s"(w2), "s"(w3), "s"(w4), "s"(w5), "s"(w6), "s"(w7), "s"(w8), "s"(w9));
}


// Optional per-launch timing (off by default; see rtp_profile_enable).  When enabled, the launch made
// inside the scope is bracketed by two timing events on its own stream and booked under `name` with its
// algorithmic flops / bytes.
struct ProfileScope {
  ProfileScope(hipStream_t stream, const char* name, double flops, double bytes);
  ~ProfileScope();
  // With device time stamps switched on (rtp_profile_enable(2)): books this launch and returns the address of its
  // two-word stamp slot for the kernel to fill (earliest start, latest end of the wall clock); otherwise null.
  unsigned long long* trace_slot();
  ProfileScope(const ProfileScope&) = delete;
  ProfileScope& operator=(const ProfileScope&) = delete;

 private:
  hipStream_t stream_;
  hipEvent_t start_ = nullptr;
  const char* name_;
  double flops_, bytes_;
};

}  // namespace rtp
