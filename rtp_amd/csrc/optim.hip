// Elementwise passes over flat shard buffers: the fused clip + SGD + shadow-cast step and dtype casts.
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
