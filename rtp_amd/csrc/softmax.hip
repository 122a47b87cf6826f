// Row softmax for the attention scores, forward and backward: one wavefront per (batch*head, query)
// row, fp32 statistics by cross-lane reduction.
#include "common.h"

namespace rtp {

constexpr int kRowsPerBlock = 4;

template <typename T>
__global__ __launch_bounds__(256) void softmax_fwd_kernel(const float* s, const float* mask, const float* kbias,
                                                          long n_batch, long heads, int causal, float scale,
                                                          long rows, long l, long skv, T* p, long mask_mod,
                                                          const float* keep, T* p_dropped) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const long i = row % l;
  const float* srow = s + row * skv;
  // one [l, skv] mask for every problem, or mask_mod of them: problem z takes mask[z % mask_mod]
  const float* mrow = mask ? mask + (mask_mod > 1 ? ((row / l) % mask_mod) * l * skv : 0) + i * skv : nullptr;
  // per-(batch, key) bias: problem index row / l = (group * n_batch + batch) * heads + head
  const float* krow = kbias ? kbias + ((row / l / heads) % n_batch) * skv : nullptr;
  T* prow = p + row * skv;
  // attention dropout: keep[z,i,j] is 0 or 1 / (1 - rate); the probabilities that meet V go to p_dropped
  const float* keeprow = keep ? keep + row * skv : nullptr;
  T* pdrow = keep ? p_dropped + row * skv : nullptr;
  const long jmax = causal ? (i + (skv - l) + 1 < skv ? i + (skv - l) + 1 : skv) : skv;  // columns [0, jmax) are visible

  float mx = -INFINITY;
  for (long j = lane; j < jmax; j += kWave) {
    float v = srow[j] * scale;
    if (mrow) v += mrow[j];
    if (krow) v += krow[j];
    mx = fmaxf(mx, v);
  }
  mx = wave_max(mx);
  float sum = 0.0f;
  for (long j = lane; j < jmax; j += kWave) {
    float v = srow[j] * scale;
    if (mrow) v += mrow[j];
    if (krow) v += krow[j];
    sum += expf(v - mx);
  }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
  for (long j = lane; j < skv; j += kWave) {
    float o = 0.0f;
    if (j < jmax) {
      float v = srow[j] * scale;
      if (mrow) v += mrow[j];
      if (krow) v += krow[j];
      o = expf(v - mx) * inv;
    }
    const T rounded = from_f32<T>(o);
    prow[j] = rounded;
    if (keeprow) pdrow[j] = from_f32<T>(to_f32(rounded) * keeprow[j]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_bwd_kernel(const T* p, const float* dp, const float* keep, float scale,
                                                          long rows, long skv, T* ds) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* prow = p + row * skv;
  const float* dprow = dp + row * skv;
  T* dsrow = ds + row * skv;
  // with dropout, dp arrives as the gradient of the dropped probabilities: times keep gives that of p
  const float* keeprow = keep ? keep + row * skv : nullptr;
  float dot = 0.0f;
  for (long j = lane; j < skv; j += kWave) dot += to_f32(prow[j]) * (keeprow ? dprow[j] * keeprow[j] : dprow[j]);
  dot = wave_sum(dot);
  for (long j = lane; j < skv; j += kWave) {
    const float pv = to_f32(prow[j]);
    const float g = keeprow ? dprow[j] * keeprow[j] : dprow[j];
    dsrow[j] = from_f32<T>(scale * pv * (g - dot));
  }
}

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_softmax_fwd_masks(void* stream, int dtype, const float* s, const float* mask, int64_t mask_problems,
                                     const float* key_bias, int64_t n_batch, int64_t heads, int causal, float scale,
                                     int64_t z, int64_t l, int64_t skv, void* p, const float* keep, void* p_dropped) {
  RTP_REQUIRE(s && p, "rtp_softmax_fwd: null pointer");
  RTP_REQUIRE(!keep == !p_dropped, "rtp_softmax_fwd: keep and p_dropped go together");
  RTP_REQUIRE(mask_problems >= 0 && (mask_problems <= 1 || (mask && z % mask_problems == 0)),
              "rtp_softmax_fwd: %lld masks do not divide z=%lld problems", (long long)mask_problems, (long long)z);
  RTP_REQUIRE(!key_bias || (n_batch >= 1 && heads >= 1 && z % (n_batch * heads) == 0),
              "rtp_softmax_fwd: a key bias needs z = groups * n_batch * heads (z=%lld n_batch=%lld heads=%lld)",
              (long long)z, (long long)n_batch, (long long)heads);
  RTP_REQUIRE(z >= 0 && l >= 0 && skv >= 1, "rtp_softmax_fwd: bad shape z=%lld l=%lld s=%lld", (long long)z,
              (long long)l, (long long)skv);
  const int64_t rows = z * l;
  if (rows == 0) return RTP_OK;
  RTP_REQUIRE(ceil_div(rows, kRowsPerBlock) < (1ll << 31), "rtp_softmax_fwd: too many rows");
  dim3 grid((unsigned)ceil_div(rows, kRowsPerBlock));
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_fwd", 0.0, (double)rows * skv * (4.0 + (dtype == RTP_F32 ? 4 : 2)));
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(softmax_fwd_kernel<float>, grid, dim3(256), 0, st, s, mask, key_bias, (long)n_batch, (long)heads,
                       causal, scale, (long)rows, (long)l, (long)skv, (float*)p, (long)mask_problems, keep,
                       (float*)p_dropped);
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(softmax_fwd_kernel<bf16_t>, grid, dim3(256), 0, st, s, mask, key_bias, (long)n_batch, (long)heads,
                       causal, scale, (long)rows, (long)l, (long)skv, (bf16_t*)p, (long)mask_problems, keep,
                       (bf16_t*)p_dropped);
  else
    return fail(RTP_ERR_ARG, "rtp_softmax_fwd: unknown dtype %d", dtype);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_softmax_fwd(void* stream, int dtype, const float* s, const float* mask, const float* key_bias,
                               int64_t n_batch, int64_t heads, int causal, float scale, int64_t z, int64_t l,
                               int64_t skv, void* p) {
  return rtp_softmax_fwd_masks(stream, dtype, s, mask, 1, key_bias, n_batch, heads, causal, scale, z, l, skv, p, nullptr,
                               nullptr);
}

extern "C" int rtp_softmax_bwd(void* stream, int dtype, const void* p, const float* dp, const float* keep, float scale,
                               int64_t z, int64_t l, int64_t skv, void* ds) {
  RTP_REQUIRE(p && dp && ds, "rtp_softmax_bwd: null pointer");
  RTP_REQUIRE(z >= 0 && l >= 0 && skv >= 1, "rtp_softmax_bwd: bad shape");
  const int64_t rows = z * l;
  if (rows == 0) return RTP_OK;
  RTP_REQUIRE(ceil_div(rows, kRowsPerBlock) < (1ll << 31), "rtp_softmax_bwd: too many rows");
  dim3 grid((unsigned)ceil_div(rows, kRowsPerBlock));
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "softmax_bwd", 0.0, (double)rows * skv * (4.0 + 2.0 * (dtype == RTP_F32 ? 4 : 2)));
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(softmax_bwd_kernel<float>, grid, dim3(256), 0, st, (const float*)p, dp, keep, scale,
                       (long)rows, (long)skv, (float*)ds);
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(softmax_bwd_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)p, dp, keep, scale,
                       (long)rows, (long)skv, (bf16_t*)ds);
  else
    return fail(RTP_ERR_ARG, "rtp_softmax_bwd: unknown dtype %d", dtype);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
