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

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Optional per-launch timing (off by default; see rtp_profile_enable).  When enabled, the launch made
// inside the scope is bracketed by two timing events on its own stream and booked under `name` with its
// algorithmic flops / bytes.
struct ProfileScope {
  ProfileScope(hipStream_t stream, const char* name, double flops, double bytes);
  ~ProfileScope();
  ProfileScope(const ProfileScope&) = delete;
  ProfileScope& operator=(const ProfileScope&) = delete;

 private:
  hipStream_t stream_;
  hipEvent_t start_ = nullptr;
  const char* name_;
  double flops_, bytes_;
};

}  // namespace rtp
