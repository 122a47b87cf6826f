// Softmax cross-entropy over the vocabulary axis of the logits, forward and backward, straight from the
// 16-bit (or fp32) logits: one workgroup per token row, 16-byte loads, fp32 statistics.
//   forward : stats[r] = {m, s} with m = max_j x[r, j], s = sum_j exp(x[r, j] - m);
//             loss[r] = (m - x[r, target[r]]) + log s
//   backward: dx[r, j] = (exp(x[r, j] - m) / s - [j == target[r]]) * dloss[r * dloss_stride]
// The maximum and the sum are kept apart (not folded into one log-sum-exp) so that rows of large common
// magnitude lose no precision.
// Rows whose target equals `ignore_index` get loss 0 and gradient 0.  Any other target outside [0, cols) is an
// error of the caller (torch asserts on the device): its row's loss is NaN, which poisons every reduction over
// the rows without a synchronisation, and its gradient is 0.
// xent_reduce_kernel folds the per-row losses into their sum or their mean over the rows that are not ignored, in
// a fixed order, and leaves 1 / count for the backward pass to scale with.
// Rows the vector kernels cannot take (class counts or pitches that are not whole 16-byte vectors, more classes
// than a workgroup holds in registers) go to element-wise kernels with the same results.
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
__device__ __forceinline__ float row_loss(long t, long ignore, int cols, float mx, float sum, float xt) {
  if (t == ignore) return 0.0f;
  return (t >= 0 && t < cols) ? (mx - xt) + logf(sum) : __builtin_nanf("");
}

template <typename T, int NV>
__global__ __launch_bounds__(kXentThreads) void xent_fwd_kernel(const T* x, long ld, int cols, const long* target,
                                                                long ignore, float* loss, float2* stats) {
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
    loss[row] = row_loss(t, ignore, cols, mx, sum, (t >= 0 && t < cols) ? to_f32(xr[t]) : 0.0f);
  }
}

// Element-wise forms for any class count and alignment: three passes over the row.
template <typename T>
__global__ __launch_bounds__(kXentThreads) void xent_fwd_any_kernel(const T* x, long ld, int cols, const long* target,
                                                                    long ignore, float* loss, float2* stats) {
  __shared__ float slots[2][4];
  const long row = blockIdx.x;
  const T* xr = x + row * ld;
  float mx = -INFINITY;
  for (int c = threadIdx.x; c < cols; c += kXentThreads) mx = fmaxf(mx, to_f32(xr[c]));
  mx = block_reduce(mx, slots[0], true);
  float sum = 0.0f;
  for (int c = threadIdx.x; c < cols; c += kXentThreads) sum += expf(to_f32(xr[c]) - mx);
  sum = block_reduce(sum, slots[1], false);
  if (threadIdx.x == 0) {
    const long t = target[row];
    stats[row] = make_float2(mx, sum);
    loss[row] = row_loss(t, ignore, cols, mx, sum, (t >= 0 && t < cols) ? to_f32(xr[t]) : 0.0f);
  }
}

template <typename T>
__global__ __launch_bounds__(kXentThreads) void xent_bwd_any_kernel(const T* x, long ld, int cols, const long* target,
                                                                    long ignore, const float2* stats,
                                                                    const float* dloss, long dloss_stride,
                                                                    const float* scale, T* dx, long ld_dx) {
  const long row = blockIdx.x;
  const T* xr = x + row * ld;
  T* dr = dx + row * ld_dx;
  const long t = target[row];
  const bool live = t != ignore && t >= 0 && t < cols;
  const float2 st = stats[row];
  const float inv = 1.0f / st.y;
  const float s = live ? dloss[row * dloss_stride] * (scale ? *scale : 1.0f) : 0.0f;
  for (int c = threadIdx.x; c < cols; c += kXentThreads) {
    float g = expf(to_f32(xr[c]) - st.x) * inv;
    if (c == t) g -= 1.0f;
    dr[c] = from_f32<T>(g * s);
  }
}

// Per-row statistics from the {max, sum exp} of the row's 64-column blocks (left by the logits product's
// epilogue): one wavefront per row, blocks combined in a fixed order; loss as in xent_fwd_kernel.
__global__ __launch_bounds__(256) void xent_combine_kernel(const float2* part, long blocks, const float* tlogit,
                                                           const long* target, long ignore, long rows, long classes,
                                                           float* loss, float2* stats) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float2* pr = part + row * blocks;
  float mx = -INFINITY;
  for (long b = lane; b < blocks; b += kWave) mx = fmaxf(mx, pr[b].x);
  mx = wave_max(mx);
  float sum = 0.0f;
  for (long b = lane; b < blocks; b += kWave) sum += pr[b].y * expf(pr[b].x - mx);
  sum = wave_sum(sum);
  if (lane == 0) {
    const long t = target[row];
    stats[row] = make_float2(mx, sum);
    loss[row] = row_loss(t, ignore, (int)classes, mx, sum, (t >= 0 && t < classes) ? tlogit[row] : 0.0f);
  }
}

// out[0] = sum of loss[0..rows) (mean != 0: divided by the number of rows whose target is not `ignore`),
// scale[0] = 1 / that number (1 for a plain sum).  One workgroup, fixed summation order.
__global__ __launch_bounds__(kXentThreads) void xent_reduce_kernel(const float* loss, const long* target, long ignore,
                                                                   long rows, int mean, float* out, float* scale) {
  __shared__ float slots[2][4];
  float sum = 0.0f, cnt = 0.0f;
  for (long r = threadIdx.x; r < rows; r += kXentThreads) {
    sum += loss[r];
    cnt += target[r] != ignore ? 1.0f : 0.0f;
  }
  sum = block_reduce(sum, slots[0], false);
  cnt = block_reduce(cnt, slots[1], false);
  if (threadIdx.x == 0) {
    out[0] = mean ? sum / cnt : sum;
    scale[0] = mean ? 1.0f / cnt : 1.0f;
  }
}

template <typename T, int NV>
__global__ __launch_bounds__(kXentThreads) void xent_bwd_kernel(const T* x, long ld, int cols, const long* target,
                                                                long ignore, const float2* stats, const float* dloss,
                                                                long dloss_stride, const float* scale, T* dx, long ld_dx) {
  touch_kernel_arguments<88>();
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
  const bool live = t != ignore && t >= 0 && t < cols;
  const float2 st = stats[row];
  const float mx = st.x, inv = 1.0f / st.y;
  const float s = live ? dloss[row * dloss_stride] * (scale ? *scale : 1.0f) : 0.0f;
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

static int xent_check(const char* who, int dtype, int64_t ld, int64_t rows, int64_t cols) {
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "%s: unknown dtype %d", who, dtype);
  RTP_REQUIRE(rows >= 0 && rows < (1ll << 31) && cols >= 1 && cols < (1ll << 31) && ld >= cols,
              "%s: need rows < 2^31, 1 <= cols < 2^31 and ld >= cols", who);
  return RTP_OK;
}

// Whether the one-pass vector kernels take the rows: whole 16-byte vectors, at most 32 per thread.
static bool xent_vectors(int dtype, int64_t ld, int64_t cols, const void* x) {
  const int vec = dtype == RTP_F32 ? 4 : 8;
  return cols % vec == 0 && cols <= (int64_t)kXentMaxVectors * vec && ld % vec == 0 && (uintptr_t)x % 16 == 0;
}

extern "C" int rtp_softmax_xent_fwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                                    const int64_t* target, int64_t ignore_index, float* loss, float* stats) {
  RTP_REQUIRE(logits && target && loss && stats, "rtp_softmax_xent_fwd: null pointer");
  RTP_REQUIRE((uintptr_t)stats % 8 == 0, "rtp_softmax_xent_fwd: stats must be 8-byte aligned");
  if (int rc = xent_check("rtp_softmax_xent_fwd", dtype, ld, rows, cols)) return rc;
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_fwd", 0.0, (double)rows * cols * (dtype == RTP_F32 ? 4.0 : 2.0));
  const dim3 grid((unsigned)rows), block(kXentThreads);
  if (!xent_vectors(dtype, ld, cols, logits)) {
    if (dtype == RTP_F32)
      hipLaunchKernelGGL(xent_fwd_any_kernel<float>, grid, block, 0, st, (const float*)logits, (long)ld, (int)cols,
                         (const long*)target, (long)ignore_index, loss, (float2*)stats);
    else
      hipLaunchKernelGGL(xent_fwd_any_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)logits, (long)ld, (int)cols,
                         (const long*)target, (long)ignore_index, loss, (float2*)stats);
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  }
  const int nv = (int)ceil_div(cols / (dtype == RTP_F32 ? 4 : 8), kXentThreads);
  if (dtype == RTP_F32)
    launch_xent_fwd<float>(nv, grid, st, (const float*)logits, (long)ld, (int)cols, (const long*)target,
                           (long)ignore_index, loss, (float2*)stats);
  else
    launch_xent_fwd<bf16_t>(nv, grid, st, (const bf16_t*)logits, (long)ld, (int)cols, (const long*)target,
                            (long)ignore_index, loss, (float2*)stats);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_softmax_xent_combine(void* stream, const float* part, int64_t blocks, const float* tlogit,
                                        const int64_t* target, int64_t ignore_index, int64_t rows, float* loss,
                                        float* stats) {
  RTP_REQUIRE(part && tlogit && target && loss && stats, "rtp_softmax_xent_combine: null pointer");
  RTP_REQUIRE(rows >= 0 && rows < (1ll << 31) && blocks >= 1 && blocks < (1ll << 25),
              "rtp_softmax_xent_combine: rows %lld / blocks %lld out of range", (long long)rows, (long long)blocks);
  RTP_REQUIRE((uintptr_t)part % 8 == 0 && (uintptr_t)stats % 8 == 0, "rtp_softmax_xent_combine: 8-byte aligned pairs");
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_combine", 0.0, 8.0 * (double)rows * blocks);
  hipLaunchKernelGGL(xent_combine_kernel, dim3((unsigned)ceil_div(rows, 4)), dim3(256), 0, st, (const float2*)part,
                     (long)blocks, tlogit, (const long*)target, (long)ignore_index, (long)rows, (long)(blocks * 64), loss,
                     (float2*)stats);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_softmax_xent_reduce(void* stream, const float* loss, const int64_t* target, int64_t ignore_index,
                                       int64_t rows, int mean, float* out, float* scale) {
  RTP_REQUIRE(loss && target && out && scale, "rtp_softmax_xent_reduce: null pointer");
  RTP_REQUIRE(rows >= 0, "rtp_softmax_xent_reduce: negative row count");
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_reduce", 0.0, 12.0 * (double)rows);
  hipLaunchKernelGGL(xent_reduce_kernel, dim3(1), dim3(kXentThreads), 0, st, loss, (const long*)target, (long)ignore_index,
                     (long)rows, mean, out, scale);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_softmax_xent_bwd(void* stream, int dtype, const void* logits, int64_t ld, int64_t rows, int64_t cols,
                                    const int64_t* target, int64_t ignore_index, const float* stats, const float* dloss,
                                    int64_t dloss_stride, const float* scale, void* dlogits, int64_t ld_dlogits) {
  RTP_REQUIRE(logits && target && stats && dloss && dlogits, "rtp_softmax_xent_bwd: null pointer");
  RTP_REQUIRE((uintptr_t)stats % 8 == 0, "rtp_softmax_xent_bwd: stats must be 8-byte aligned");
  RTP_REQUIRE(dloss_stride == 0 || dloss_stride == 1, "rtp_softmax_xent_bwd: dloss_stride must be 0 or 1");
  if (int rc = xent_check("rtp_softmax_xent_bwd", dtype, ld, rows, cols)) return rc;
  if (int rc = xent_check("rtp_softmax_xent_bwd", dtype, ld_dlogits, rows, cols)) return rc;
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_xent_bwd", 0.0, 2.0 * (double)rows * cols * (dtype == RTP_F32 ? 4.0 : 2.0));
  const dim3 grid((unsigned)rows), block(kXentThreads);
  if (!xent_vectors(dtype, ld, cols, logits) || !xent_vectors(dtype, ld_dlogits, cols, dlogits)) {
    if (dtype == RTP_F32)
      hipLaunchKernelGGL(xent_bwd_any_kernel<float>, grid, block, 0, st, (const float*)logits, (long)ld, (int)cols,
                         (const long*)target, (long)ignore_index, (const float2*)stats, dloss, (long)dloss_stride, scale, (float*)dlogits,
                         (long)ld_dlogits);
    else
      hipLaunchKernelGGL(xent_bwd_any_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)logits, (long)ld, (int)cols,
                         (const long*)target, (long)ignore_index, (const float2*)stats, dloss, (long)dloss_stride, scale, (bf16_t*)dlogits,
                         (long)ld_dlogits);
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  }
  const int nv = (int)ceil_div(cols / (dtype == RTP_F32 ? 4 : 8), kXentThreads);
  if (dtype == RTP_F32)
    launch_xent_bwd<float>(nv, grid, st, (const float*)logits, (long)ld, (int)cols, (const long*)target,
                           (long)ignore_index, (const float2*)stats, dloss, (long)dloss_stride, scale, (float*)dlogits, (long)ld_dlogits);
  else
    launch_xent_bwd<bf16_t>(nv, grid, st, (const bf16_t*)logits, (long)ld, (int)cols, (const long*)target,
                            (long)ignore_index, (const float2*)stats, dloss, (long)dloss_stride, scale, (bf16_t*)dlogits, (long)ld_dlogits);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
