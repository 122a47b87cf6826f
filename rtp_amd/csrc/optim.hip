// Elementwise passes over flat shard buffers: the fused clip + SGD + shadow-cast step and dtype casts.
#include <cmath>

#include "common.h"

namespace rtp {

template <typename T>
__global__ __launch_bounds__(256) void sgd_kernel(float* master, const T* grad, T* shadow, long n, float lr,
                                                  float clip) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float g = to_f32(grad[i]);
    if (clip > 0.0f) g = fminf(fmaxf(g, -clip), clip);
    // two roundings (product, then difference): the plain closed form w - lr*g, not a fused multiply-add
    float w;
    {
#pragma clang fp contract(off)
      const float step = lr * g;
      w = master[i] - step;
    }
    master[i] = w;
    if (shadow) shadow[i] = from_f32<T>(w);
  }
}

// Four parameters per lane and access: 16-byte master accesses, 8- or 16-byte gradient / shadow accesses; two
// such groups are loaded before either is used, so each lane keeps four loads in flight.
template <typename T>
struct Sgd4 {
  union Pack {
    T e[4];
    uint2 u2;
    uint4 u4;
  };
  static __device__ __forceinline__ Pack load(const T* p, long i) {
    Pack v;
    if (sizeof(T) == 2)
      v.u2 = nt_load(reinterpret_cast<const uint2*>(p) + i);
    else
      v.u4 = nt_load(reinterpret_cast<const uint4*>(p) + i);
    return v;
  }
  static __device__ __forceinline__ void store(T* p, long i, const Pack& v) {
    if (sizeof(T) == 2)
      nt_store(v.u2, reinterpret_cast<uint2*>(p) + i);
    else
      nt_store(v.u4, reinterpret_cast<uint4*>(p) + i);
  }
  static __device__ __forceinline__ void update(float4& w, const Pack& g, Pack& sh, float lr, float clip) {
    float* wf = reinterpret_cast<float*>(&w);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float gv = to_f32(g.e[e]);
      if (clip > 0.0f) gv = fminf(fmaxf(gv, -clip), clip);
      {
#pragma clang fp contract(off)
        const float step = lr * gv;
        wf[e] = wf[e] - step;
      }
      sh.e[e] = from_f32<T>(wf[e]);
    }
  }
};

template <typename T>
__global__ __launch_bounds__(256) void sgd_vec4_kernel(float4* master, const T* grad, T* shadow, long n4, float lr,
                                                       float clip) {
  using P = typename Sgd4<T>::Pack;
  const long stride = (long)gridDim.x * blockDim.x;
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + stride < n4; i += 2 * stride) {
    const P g0 = Sgd4<T>::load(grad, i), g1 = Sgd4<T>::load(grad, i + stride);
    float4 w0 = nt_load(master + i), w1 = nt_load(master + i + stride);
    P s0, s1;
    Sgd4<T>::update(w0, g0, s0, lr, clip);
    Sgd4<T>::update(w1, g1, s1, lr, clip);
    nt_store(w0, master + i);
    nt_store(w1, master + i + stride);
    if (shadow) {
      Sgd4<T>::store(shadow, i, s0);
      Sgd4<T>::store(shadow, i + stride, s1);
    }
  }
  for (; i < n4; i += stride) {
    const P g0 = Sgd4<T>::load(grad, i);
    float4 w0 = master[i];
    P s0;
    Sgd4<T>::update(w0, g0, s0, lr, clip);
    master[i] = w0;
    if (shadow) Sgd4<T>::store(shadow, i, s0);
  }
}

// Many tensors in one launch: workgroup b updates chunk b of a device-resident table, four parameters per lane
// and access, two accesses in flight.
struct SgdChunk {
  float* master;
  const void* grad;
  void* shadow;  // may be null
  long n;        // parameters in the chunk, a multiple of 4; the three pointers are 16-byte aligned
};

template <typename T>
__global__ __launch_bounds__(256) void sgd_multi_kernel(const SgdChunk* chunks, float lr, float clip) {
  using P = typename Sgd4<T>::Pack;
  const SgdChunk c = chunks[blockIdx.x];
  float4* master = reinterpret_cast<float4*>(c.master);
  const T* grad = reinterpret_cast<const T*>(c.grad);
  T* shadow = reinterpret_cast<T*>(c.shadow);
  const long n4 = c.n >> 2;
  long i = threadIdx.x;
  for (; i + 256 < n4; i += 512) {
    const P g0 = Sgd4<T>::load(grad, i), g1 = Sgd4<T>::load(grad, i + 256);
    float4 w0 = nt_load(master + i), w1 = nt_load(master + i + 256);
    P s0, s1;
    Sgd4<T>::update(w0, g0, s0, lr, clip);
    Sgd4<T>::update(w1, g1, s1, lr, clip);
    nt_store(w0, master + i);
    nt_store(w1, master + i + 256);
    if (shadow) {
      Sgd4<T>::store(shadow, i, s0);
      Sgd4<T>::store(shadow, i + 256, s1);
    }
  }
  for (; i < n4; i += 256) {
    const P g0 = Sgd4<T>::load(grad, i);
    float4 w0 = nt_load(master + i);
    P s0;
    Sgd4<T>::update(w0, g0, s0, lr, clip);
    nt_store(w0, master + i);
    if (shadow) Sgd4<T>::store(shadow, i, s0);
  }
}

// Adam on a flat buffer.  The arithmetic follows torch.optim.Adam's single-tensor form step by step, each
// operation rounded on its own.
struct AdamScalars {
  float w1, beta2, w2, bc2_sqrt, eps, neg_step_size, weight_decay, clip;  // w1 = 1 - beta1, w2 = 1 - beta2
  // step count in device memory (or null): bc2_sqrt and neg_step_size are then formed by the kernel, so that a
  // replayed graph moves on with the caller's counter
  const long* step_dev;
  double lr, beta1, beta2d;
};
__device__ __forceinline__ void adam_bias_corrections(AdamScalars& c) {
  if (!c.step_dev) return;
  const double t = (double)*c.step_dev;
  const double bc1 = 1.0 - pow(c.beta1, t), bc2 = 1.0 - pow(c.beta2d, t);
  c.bc2_sqrt = (float)sqrt(bc2);
  c.neg_step_size = (float)(-(c.lr / bc1));
}
__device__ __forceinline__ void adam_update(float& w, float& m, float& v, float g, const AdamScalars& c) {
#pragma clang fp contract(off)
  if (c.clip > 0.0f) g = fminf(fmaxf(g, -c.clip), c.clip);
  if (c.weight_decay != 0.0f) g = g + c.weight_decay * w;
  m = m + c.w1 * (g - m);            // exp_avg.lerp_(grad, 1 - beta1)
  v = v * c.beta2 + (c.w2 * g) * g;  // exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value = 1 - beta2)
  const float denom = sqrtf(v) / c.bc2_sqrt + c.eps;
  w = w + c.neg_step_size * (m / denom);  // param.addcdiv_(exp_avg, denom, value = -step_size)
}

template <typename T>
__global__ __launch_bounds__(256) void adam_kernel(float* master, const T* grad, T* shadow, float* exp_avg,
                                                   float* exp_avg_sq, long n, AdamScalars c) {
  adam_bias_corrections(c);
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    float w = master[i], m = exp_avg[i], v = exp_avg_sq[i];
    adam_update(w, m, v, to_f32(grad[i]), c);
    master[i] = w, exp_avg[i] = m, exp_avg_sq[i] = v;
    if (shadow) shadow[i] = from_f32<T>(w);
  }
}

// Four parameters per lane and access, streaming (non-temporal) 16-byte accesses to the three fp32 arrays, two
// groups in flight per lane.
template <typename T>
__global__ __launch_bounds__(256) void adam_vec4_kernel(float4* master, const T* grad, T* shadow, float4* exp_avg,
                                                        float4* exp_avg_sq, long n4, AdamScalars c) {
  using P = typename Sgd4<T>::Pack;
  adam_bias_corrections(c);
  const long stride = (long)gridDim.x * blockDim.x;
  auto update4 = [&](float4& w, float4& m, float4& v, const P& g, P& sh) {
    float *wf = reinterpret_cast<float*>(&w), *mf = reinterpret_cast<float*>(&m), *vf = reinterpret_cast<float*>(&v);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      adam_update(wf[e], mf[e], vf[e], to_f32(g.e[e]), c);
      sh.e[e] = from_f32<T>(wf[e]);
    }
  };
  long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + stride < n4; i += 2 * stride) {
    const long k = i + stride;
    const P g0 = Sgd4<T>::load(grad, i), g1 = Sgd4<T>::load(grad, k);
    float4 w0 = nt_load(master + i), w1 = nt_load(master + k);
    float4 m0 = nt_load(exp_avg + i), m1 = nt_load(exp_avg + k);
    float4 v0 = nt_load(exp_avg_sq + i), v1 = nt_load(exp_avg_sq + k);
    P s0, s1;
    update4(w0, m0, v0, g0, s0);
    update4(w1, m1, v1, g1, s1);
    nt_store(w0, master + i), nt_store(w1, master + k);
    nt_store(m0, exp_avg + i), nt_store(m1, exp_avg + k);
    nt_store(v0, exp_avg_sq + i), nt_store(v1, exp_avg_sq + k);
    if (shadow) {
      Sgd4<T>::store(shadow, i, s0);
      Sgd4<T>::store(shadow, k, s1);
    }
  }
  for (; i < n4; i += stride) {
    const P g0 = Sgd4<T>::load(grad, i);
    float4 w0 = master[i], m0 = exp_avg[i], v0 = exp_avg_sq[i];
    P s0;
    update4(w0, m0, v0, g0, s0);
    master[i] = w0, exp_avg[i] = m0, exp_avg_sq[i] = v0;
    if (shadow) Sgd4<T>::store(shadow, i, s0);
  }
}

// Adam for many buffers in one launch: workgroup b updates chunk b of a device-resident table.
struct AdamChunk {
  float* master;
  const void* grad;
  void* shadow;  // may be null
  float *exp_avg, *exp_avg_sq;
  long n;  // parameters in the chunk, a multiple of 4; the pointers are 16-byte aligned
};
template <typename T>
__global__ __launch_bounds__(256) void adam_multi_kernel(const AdamChunk* chunks, AdamScalars c) {
  using P = typename Sgd4<T>::Pack;
  adam_bias_corrections(c);
  const AdamChunk ch = chunks[blockIdx.x];
  float4* master = reinterpret_cast<float4*>(ch.master);
  float4* m4 = reinterpret_cast<float4*>(ch.exp_avg);
  float4* v4 = reinterpret_cast<float4*>(ch.exp_avg_sq);
  const T* grad = reinterpret_cast<const T*>(ch.grad);
  T* shadow = reinterpret_cast<T*>(ch.shadow);
  const long n4 = ch.n >> 2;
  auto one = [&](long i, const P& g, float4 w, float4 m, float4 v) {
    float *wf = reinterpret_cast<float*>(&w), *mf = reinterpret_cast<float*>(&m), *vf = reinterpret_cast<float*>(&v);
    P sh;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      adam_update(wf[e], mf[e], vf[e], to_f32(g.e[e]), c);
      sh.e[e] = from_f32<T>(wf[e]);
    }
    nt_store(w, master + i), nt_store(m, m4 + i), nt_store(v, v4 + i);
    if (shadow) Sgd4<T>::store(shadow, i, sh);
  };
  long i = threadIdx.x;
  for (; i + 256 < n4; i += 512) {
    const long k = i + 256;
    const P g0 = Sgd4<T>::load(grad, i), g1 = Sgd4<T>::load(grad, k);
    const float4 w0 = nt_load(master + i), w1 = nt_load(master + k);
    const float4 a0 = nt_load(m4 + i), a1 = nt_load(m4 + k);
    const float4 b0 = nt_load(v4 + i), b1 = nt_load(v4 + k);
    one(i, g0, w0, a0, b0);
    one(k, g1, w1, a1, b1);
  }
  for (; i < n4; i += 256) one(i, Sgd4<T>::load(grad, i), nt_load(master + i), nt_load(m4 + i), nt_load(v4 + i));
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S* src, D* dst, long n) {
  const long stride = (long)gridDim.x * blockDim.x;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = from_f32<D>(to_f32(src[i]));
}

static unsigned flat_grid(int64_t n) { return (unsigned)std::min<int64_t>(4096, std::max<int64_t>(1, ceil_div(n, 1024))); }

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_sgd_step(void* stream, int dtype, float* master, const void* grad, void* shadow, int64_t n,
                            float lr, float clip) {
  RTP_REQUIRE(master && grad, "rtp_sgd_step: null pointer");
  RTP_REQUIRE(n >= 0, "rtp_sgd_step: negative length");
  if (n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t tsz = dtype == RTP_F32 ? 4 : 2;
  const bool vec4 = n % 4 == 0 && (uintptr_t)master % 16 == 0 && (uintptr_t)grad % (4 * tsz) == 0 &&
                    (!shadow || (uintptr_t)shadow % (4 * tsz) == 0);
  ProfileScope prof(s, "sgd_step", 2.0 * (double)n, (double)n * (8.0 + (dtype == RTP_F32 ? 4 : 2) * (shadow ? 2.0 : 1.0)));
  if (dtype != RTP_F32 && dtype != RTP_BF16) return fail(RTP_ERR_ARG, "rtp_sgd_step: unknown dtype %d", dtype);
  if (vec4 && dtype == RTP_F32)
    hipLaunchKernelGGL(sgd_vec4_kernel<float>, dim3(flat_grid(n / 4)), dim3(256), 0, s, (float4*)master,
                       (const float*)grad, (float*)shadow, (long)(n / 4), lr, clip);
  else if (vec4)
    hipLaunchKernelGGL(sgd_vec4_kernel<bf16_t>, dim3(flat_grid(n / 4)), dim3(256), 0, s, (float4*)master,
                       (const bf16_t*)grad, (bf16_t*)shadow, (long)(n / 4), lr, clip);
  else if (dtype == RTP_F32)
    hipLaunchKernelGGL(sgd_kernel<float>, dim3(flat_grid(n)), dim3(256), 0, s, master, (const float*)grad,
                       (float*)shadow, (long)n, lr, clip);
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(sgd_kernel<bf16_t>, dim3(flat_grid(n)), dim3(256), 0, s, master, (const bf16_t*)grad,
                       (bf16_t*)shadow, (long)n, lr, clip);
  else
    return fail(RTP_ERR_ARG, "rtp_sgd_step: unknown dtype %d", dtype);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_sgd_step_multi(void* stream, int dtype, const rtp_sgd_chunk* chunks, int64_t n_chunks, float lr,
                                  float clip, double total_params) {
  static_assert(sizeof(rtp_sgd_chunk) == sizeof(SgdChunk), "rtp_sgd_chunk layout");
  RTP_REQUIRE(chunks, "rtp_sgd_step_multi: null chunk table");
  RTP_REQUIRE(n_chunks >= 0 && n_chunks < (1ll << 31), "rtp_sgd_step_multi: chunk count %lld out of range",
              (long long)n_chunks);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_sgd_step_multi: unknown dtype %d", dtype);
  if (n_chunks == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  ProfileScope prof(s, "sgd_step", 2.0 * total_params, total_params * (dtype == RTP_F32 ? 12.0 : 12.0));
  const SgdChunk* table = reinterpret_cast<const SgdChunk*>(chunks);
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(sgd_multi_kernel<float>, dim3((unsigned)n_chunks), dim3(256), 0, s, table, lr, clip);
  else
    hipLaunchKernelGGL(sgd_multi_kernel<bf16_t>, dim3((unsigned)n_chunks), dim3(256), 0, s, table, lr, clip);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

template <typename T>
static void launch_adam(hipStream_t s, bool vec4, float* master, const void* grad, void* shadow, float* exp_avg,
                        float* exp_avg_sq, int64_t n, const AdamScalars& c) {
  if (vec4)
    hipLaunchKernelGGL(adam_vec4_kernel<T>, dim3(flat_grid(n / 4)), dim3(256), 0, s, (float4*)master, (const T*)grad,
                       (T*)shadow, (float4*)exp_avg, (float4*)exp_avg_sq, (long)(n / 4), c);
  else
    hipLaunchKernelGGL(adam_kernel<T>, dim3(flat_grid(n)), dim3(256), 0, s, master, (const T*)grad, (T*)shadow, exp_avg,
                       exp_avg_sq, (long)n, c);
}

extern "C" int rtp_adam_step(void* stream, int dtype, float* master, const void* grad, void* shadow, float* exp_avg,
                             float* exp_avg_sq, int64_t n, double lr, double beta1, double beta2, double eps,
                             double weight_decay, int64_t step, const int64_t* step_dev, double clip) {
  RTP_REQUIRE(master && grad && exp_avg && exp_avg_sq, "rtp_adam_step: null pointer");
  RTP_REQUIRE(n >= 0, "rtp_adam_step: negative length");
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_adam_step: unknown dtype %d", dtype);
  RTP_REQUIRE(step_dev || step >= 1, "rtp_adam_step: step counts from 1 (got %lld)", (long long)step);
  RTP_REQUIRE(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0 && eps >= 0.0 && lr >= 0.0,
              "rtp_adam_step: need 0 <= beta < 1, eps >= 0, lr >= 0");
  if (n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  // the scalars are formed in double as the Python optimiser does, then applied in fp32
  const double t = step_dev ? 1.0 : (double)step;
  const double bc1 = 1.0 - std::pow(beta1, t), bc2 = 1.0 - std::pow(beta2, t);
  AdamScalars c{};
  c.step_dev = reinterpret_cast<const long*>(step_dev), c.lr = lr, c.beta1 = beta1, c.beta2d = beta2;
  c.w1 = (float)(1.0 - beta1), c.beta2 = (float)beta2, c.w2 = (float)(1.0 - beta2);
  c.bc2_sqrt = (float)std::sqrt(bc2), c.eps = (float)eps, c.neg_step_size = (float)(-(lr / bc1));
  c.weight_decay = (float)weight_decay, c.clip = (float)clip;
  const size_t tsz = dtype == RTP_F32 ? 4 : 2;
  const bool vec4 = n % 4 == 0 && ((uintptr_t)master | (uintptr_t)exp_avg | (uintptr_t)exp_avg_sq) % 16 == 0 &&
                    (uintptr_t)grad % (4 * tsz) == 0 && (!shadow || (uintptr_t)shadow % (4 * tsz) == 0);
  ProfileScope prof(s, "adam_step", 12.0 * (double)n, (double)n * (24.0 + tsz * (shadow ? 2.0 : 1.0)));
  if (dtype == RTP_F32)
    launch_adam<float>(s, vec4, master, grad, shadow, exp_avg, exp_avg_sq, n, c);
  else
    launch_adam<bf16_t>(s, vec4, master, grad, shadow, exp_avg, exp_avg_sq, n, c);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_adam_step_multi(void* stream, int dtype, const rtp_adam_chunk* chunks, int64_t n_chunks, double lr,
                                   double beta1, double beta2, double eps, double weight_decay, int64_t step,
                                   const int64_t* step_dev, double clip, double total_params) {
  static_assert(sizeof(rtp_adam_chunk) == sizeof(AdamChunk), "rtp_adam_chunk layout");
  RTP_REQUIRE(chunks, "rtp_adam_step_multi: null chunk table");
  RTP_REQUIRE(n_chunks >= 0 && n_chunks < (1ll << 31), "rtp_adam_step_multi: chunk count %lld out of range",
              (long long)n_chunks);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_adam_step_multi: unknown dtype %d", dtype);
  RTP_REQUIRE(step_dev || step >= 1, "rtp_adam_step_multi: step counts from 1 (got %lld)", (long long)step);
  RTP_REQUIRE(beta1 >= 0.0 && beta1 < 1.0 && beta2 >= 0.0 && beta2 < 1.0 && eps >= 0.0 && lr >= 0.0,
              "rtp_adam_step_multi: need 0 <= beta < 1, eps >= 0, lr >= 0");
  if (n_chunks == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  const double t = step_dev ? 1.0 : (double)step;
  const double bc1 = 1.0 - std::pow(beta1, t), bc2 = 1.0 - std::pow(beta2, t);
  AdamScalars c{};
  c.step_dev = reinterpret_cast<const long*>(step_dev), c.lr = lr, c.beta1 = beta1, c.beta2d = beta2;
  c.w1 = (float)(1.0 - beta1), c.beta2 = (float)beta2, c.w2 = (float)(1.0 - beta2);
  c.bc2_sqrt = (float)std::sqrt(bc2), c.eps = (float)eps, c.neg_step_size = (float)(-(lr / bc1));
  c.weight_decay = (float)weight_decay, c.clip = (float)clip;
  ProfileScope prof(s, "adam_step", 12.0 * total_params, total_params * (dtype == RTP_F32 ? 32.0 : 28.0));
  const AdamChunk* table = reinterpret_cast<const AdamChunk*>(chunks);
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(adam_multi_kernel<float>, dim3((unsigned)n_chunks), dim3(256), 0, s, table, c);
  else
    hipLaunchKernelGGL(adam_multi_kernel<bf16_t>, dim3((unsigned)n_chunks), dim3(256), 0, s, table, c);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_cast(void* stream, int dtype_src, const void* src, int dtype_dst, void* dst, int64_t n) {
  RTP_REQUIRE(src && dst, "rtp_cast: null pointer");
  RTP_REQUIRE(n >= 0, "rtp_cast: negative length");
  if (n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(flat_grid(n));
  if (dtype_src == RTP_F32 && dtype_dst == RTP_BF16)
    hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, dim3(256), 0, s, (const float*)src, (bf16_t*)dst, (long)n);
  else if (dtype_src == RTP_BF16 && dtype_dst == RTP_F32)
    hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, dim3(256), 0, s, (const bf16_t*)src, (float*)dst, (long)n);
  else if (dtype_src == RTP_F32 && dtype_dst == RTP_F32)
    hipLaunchKernelGGL((cast_kernel<float, float>), grid, dim3(256), 0, s, (const float*)src, (float*)dst, (long)n);
  else if (dtype_src == RTP_BF16 && dtype_dst == RTP_BF16)
    hipLaunchKernelGGL((cast_kernel<bf16_t, bf16_t>), grid, dim3(256), 0, s, (const bf16_t*)src, (bf16_t*)dst, (long)n);
  else
    return fail(RTP_ERR_ARG, "rtp_cast: unknown dtype pair %d -> %d", dtype_src, dtype_dst);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
