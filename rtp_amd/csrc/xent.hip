// Softmax cross-entropy over the vocabulary axis of the logits, forward and backward, straight from the
// 16-bit (or fp32) logits: one workgroup per token row, 16-byte loads, fp32 statistics.
//   forward : stats[r] = {m, s} with m = max_j x[r, j], s = sum_j exp(x[r, j] - m);
//             loss[r] = (m - x[r, target[r]]) + log s
//   backward: dx[r, j] = (exp(x[r, j] - m) / s - [j == target[r]]) * dloss[r * dloss_stride]
// The maximum and the sum are kept apart (not folded into one log-sum-exp) so that rows of large common
// magnitude lose no precision.
// Rows whose target is outside [0, cols) (an ignore index) get loss 0 and gradient 0.
#include "common.h"

namespace rtp {

constexpr int kXentThreads = 256;

template <typename T>
struct XVec {
  static constexpr int N = 16 / sizeof(T);
  union {
    uint4 q;
    T e[N];
  };
};

__device__ __forceinline__ float block_reduce(float v, float* slot, bool is_max) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, kWave);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
  __syncthreads();
  return is_max ? fmaxf(fmaxf(slot[0], slot[1]), fmaxf(slot[2], slot[3])) : (slot[0] + slot[1]) + (slot[2] + slot[3]);
}

// NV: 16-byte vectors per thread (the row has at most NV * 256 of them).  Every vector of the row is requested
// before the first one is used and stays in registers for the second pass: a thread that loads in a loop waits out
// one trip to memory per iteration, and the row would be read twice.
template <typename T, int NV>
__global__ __launch_bounds__(kXentThreads) void xent_fwd_kernel(const T* x, long ld, int cols, const long* target,
                                                                float* loss, float2* stats) {
  constexpr int VEC = XVec<T>::N;
  __shared__ float slots[2][4];
  const long row = blockIdx.x;
  const T* xr = x + row * ld;
  const int nvec = cols / VEC;  // cols is a multiple of VEC
  XVec<T> v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kXentThreads;
    v[i].q = reinterpret_cast<const uint4*>(xr)[c < nvec ? c : 0];
  }
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if (threadIdx.x + i * kXentThreads < nvec) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) mx = fmaxf(mx, to_f32(v[i].e[e]));
    }
  mx = block_reduce(mx, slots[0], true);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
    if (threadIdx.x + i * kXentThreads < nvec) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum += expf(to_f32(v[i].e[e]) - mx);
    }
  sum = block_reduce(sum, slots[1], false);
  if (threadIdx.x == 0) {
    const long t = target[row];
    stats[row] = make_float2(mx, sum);
    loss[row] = (t >= 0 && t < cols) ? (mx - to_f32(xr[t])) + logf(sum) : 0.0f;
  }
}

template <typename T, int NV>
__global__ __launch_bounds__(kXentThreads) void xent_bwd_kernel(const T* x, long ld, int cols, const long* target,
                                                                const float2* stats, const float* dloss, long dloss_stride,
                                                                T* dx, long ld_dx) {
  touch_kernel_arguments<72>();
  constexpr int VEC = XVec<T>::N;
  const long row = blockIdx.x;
  const T* xr = x + row * ld;
  T* dr = dx + row * ld_dx;
  const int nvec = cols / VEC;
  XVec<T> v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kXentThreads;
    v[i].q = reinterpret_cast<const uint4*>(xr)[c < nvec ? c : 0];
  }
  const long t = target[row];
  const bool live = t >= 0 && t < cols;
  const float2 st = stats[row];
  const float mx = st.x, inv = 1.0f / st.y;
  const float s = live ? dloss[row * dloss_stride] : 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kXentThreads;
    if (c < nvec) {
      XVec<T> o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float g = expf(to_f32(v[i].e[e]) - mx) * inv;
        if ((long)c * VEC + e == t) g -= 1.0f;
        o.e[e] = from_f32<T>(g * s);
      }
      reinterpret_cast<uint4*>(dr)[c] = o.q;
    }
  }
}

// The kernels are instantiated for 1, 2, 4, 8, 16 and 32 vectors per thread: rows of up to 65536 16-bit classes.
constexpr int kXentMaxVectors = 32 * kXentThreads;

template <typename T, typename... Args>
static void launch_xent_fwd(int nv, dim3 grid, hipStream_t st, Args... args) {
  const dim3 block(kXentThreads);
  if (nv <= 1) hipLaunchKernelGGL((xent_fwd_kernel<T, 1>), grid, block, 0, st, args...);
  else if (nv <= 2) hipLaunchKernelGGL((xent_fwd_kernel<T, 2>), grid, block, 0, st, args...);
  else if (nv <= 4) hipLaunchKernelGGL((xent_fwd_kernel<T, 4>), grid, block, 0, st, args...);
  else if (nv <= 8) hipLaunchKernelGGL((xent_fwd_kernel<T, 8>), grid, block, 0, st, args...);
  else if (nv <= 16) hipLaunchKernelGGL((xent_fwd_kernel<T, 16>), grid, block, 0, st, args...);
  else hipLaunchKernelGGL((xent_fwd_kernel<T, 32>), grid, block, 0, st, args...);
}
template <typename T, typename... Args>
static void launch_xent_bwd(int nv, dim3 grid, hipStream_t st, Args... args) {
  const dim3 block(kXentThreads);
  if (nv <= 1) hipLaunchKernelGGL((xent_bwd_kernel<T, 1>), grid, block, 0, st, args...);
  else if (nv <= 2) hipLaunchKernelGGL((xent_bwd_kernel<T, 2>), grid, block, 0, st, args...);
  else if (nv <= 4) hipLaunchKernelGGL((xent_bwd_kernel<T, 4>), grid, block, 0, st, args...);
  else if (nv <= 8) hipLaunchKernelGGL((xent_bwd_kernel<T, 8>), grid, block, 0, st, args...);
  else if (nv <= 16) hipLaunchKernelGGL((xent_bwd_kernel<T, 16>), grid, block, 0, st, args...);
  else hipLaunchKernelGGL((xent_bwd_kernel<T, 32>), grid, block, 0, st, args...);
}

}  // namespace rtp

using namespace rtp;

static int xent_check(const char* who, int dtype, int64_t ld, int64_t rows, int64_t cols, const void* x) {
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "%s: unknown dtype %d", who, dtype);
  const int vec = dtype == RTP_F32 ? 4 : 8;
  RTP_REQUIRE(rows >= 0 && rows < (1ll << 31) && cols >= vec && cols <= (int64_t)kXentMaxVectors * vec &&
                  cols % vec == 0 && ld >= cols && ld % vec == 0 && (uintptr_t)x % 16 == 0,
              "%s: need rows < 2^31, cols a multiple of %d and at most %d, ld >= cols and a multiple of %d, 16-byte "
              "aligned logits",
              who, vec, kXentMaxVectors * vec, vec);
  return RTP_OK;
}

extern "C" int rtp_softmax_xent_fwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                                    const int64_t* target, float* loss, float* stats) {
  RTP_REQUIRE(logits && target && loss && stats, "rtp_softmax_xent_fwd: null pointer");
  RTP_REQUIRE((uintptr_t)stats % 8 == 0, "rtp_softmax_xent_fwd: stats must be 8-byte aligned");
  if (int rc = xent_check("rtp_softmax_xent_fwd", dtype, ld, rows, cols, logits)) return rc;
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_fwd", 0.0, (double)rows * cols * (dtype == RTP_F32 ? 4.0 : 2.0));
  const int nv = (int)ceil_div(cols / (dtype == RTP_F32 ? 4 : 8), kXentThreads);
  if (dtype == RTP_F32)
    launch_xent_fwd<float>(nv, dim3((unsigned)rows), st, (const float*)logits, (long)ld, (int)cols, (const long*)target, loss,
                           (float2*)stats);
  else
    launch_xent_fwd<bf16_t>(nv, dim3((unsigned)rows), st, (const bf16_t*)logits, (long)ld, (int)cols, (const long*)target,
                            loss, (float2*)stats);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_softmax_xent_bwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                                    const int64_t* target, const float* stats, const float* dloss, int64_t dloss_stride,
                                    void* dlogits, int64_t ld_dlogits) {
  RTP_REQUIRE(logits && target && stats && dloss && dlogits, "rtp_softmax_xent_bwd: null pointer");
  RTP_REQUIRE((uintptr_t)stats % 8 == 0, "rtp_softmax_xent_bwd: stats must be 8-byte aligned");
  RTP_REQUIRE(dloss_stride == 0 || dloss_stride == 1, "rtp_softmax_xent_bwd: dloss_stride must be 0 or 1");
  if (int rc = xent_check("rtp_softmax_xent_bwd", dtype, ld, rows, cols, logits)) return rc;
  if (int rc = xent_check("rtp_softmax_xent_bwd", dtype, ld_dlogits, rows, cols, dlogits)) return rc;
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_bwd", 0.0, 2.0 * (double)rows * cols * (dtype == RTP_F32 ? 4.0 : 2.0));
  const int nv = (int)ceil_div(cols / (dtype == RTP_F32 ? 4 : 8), kXentThreads);
  if (dtype == RTP_F32)
    launch_xent_bwd<float>(nv, dim3((unsigned)rows), st, (const float*)logits, (long)ld, (int)cols, (const long*)target,
                           (const float2*)stats, dloss, (long)dloss_stride, (float*)dlogits, (long)ld_dlogits);
  else
    launch_xent_bwd<bf16_t>(nv, dim3((unsigned)rows), st, (const bf16_t*)logits, (long)ld, (int)cols, (const long*)target,
                            (const float2*)stats, dloss, (long)dloss_stride, (bf16_t*)dlogits, (long)ld_dlogits);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
