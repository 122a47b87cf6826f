// Gate projection of the MoE layer: logits[S, E] = x[S, M] wg[E, M]^T with a handful of experts (E <= 16), its
// input gradient and its weight gradient.  With so few output columns these are streaming passes over x (or dx),
// bound by memory, not matrix products worth a tile: the expert rows of wg stay in registers / L1 and every
// token row is read (or written) once.
#include "common.h"

#include <mutex>

#include "rtp_hip.h"

namespace rtp {

constexpr int kGateMaxExperts = 16;
constexpr int kGateFwdRows = 4;     // token rows per wavefront in the forward kernel
constexpr int kGateDgradRows = 16;  // token rows per workgroup in the input-gradient kernel
constexpr int kGateWgradRows = 64;  // token rows per partial sum of the weight gradient

template <typename T>
struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  union {
    uint4 q;
    T e[N];
  };
};

// All three kernels are instantiated for EB = 4, 8 or 16 expert slots (the smallest that holds E) and are branch-free
// over the slots: a slot beyond E re-reads expert 0 and its result is dropped or weighted by zero.  A test per expert
// would split the code into one block per expert, each with its own trip to memory before its arithmetic.

// logits[s][e] = sum_m x[s][m] * w[e][m], fp32.  One wavefront per kGateFwdRows token rows: a lane owns the m-vectors
// lane, lane + 64, ... of every row, each expert vector is loaded once per m-vector and used for all the rows.
template <typename T, int EB>
__global__ __launch_bounds__(256) void gate_fwd_kernel(const T* x, long ldx, const T* w, long ldw, long S, int M, int E,
                                                       float* logits, long ldl) {
  constexpr int VEC = Vec16<T>::N, R = kGateFwdRows;
  const int lane = threadIdx.x & 63;
  const long row0 = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
  if (row0 >= S) return;
  float acc[R][EB];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < EB; ++e) acc[r][e] = 0.0f;
  const T* xr[R];
#pragma unroll
  for (int r = 0; r < R; ++r) xr[r] = x + (row0 + r < S ? row0 + r : S - 1) * ldx;  // rows outside: recomputed, not stored
  const T* wr[EB];
#pragma unroll
  for (int e = 0; e < EB; ++e) wr[e] = w + (e < E ? e : 0) * ldw;
  for (int c = lane; c < M / VEC; c += kWave) {
    Vec16<T> xv[R], wv[EB];
#pragma unroll
    for (int r = 0; r < R; ++r) xv[r].q = *reinterpret_cast<const uint4*>(xr[r] + c * VEC);
#pragma unroll
    for (int e = 0; e < EB; ++e) wv[e].q = *reinterpret_cast<const uint4*>(wr[e] + c * VEC);
#pragma unroll
    for (int e = 0; e < EB; ++e)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int k = 0; k < VEC; ++k) acc[r][e] += to_f32(xv[r].e[k]) * to_f32(wv[e].e[k]);
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int e = 0; e < EB; ++e) {
      const float v = wave_sum(acc[r][e]);
      if (lane == 0 && row0 + r < S && e < E) logits[(row0 + r) * ldl + e] = v;
    }
}

// The block of dl that a workgroup needs, rows [s0, s0 + ROWS) x EB slots, zero outside S x E, into LDS in one batch.
template <int ROWS, int EB>
__device__ __forceinline__ void stage_dl(const float* dl, long ldl, long s0, long S, int E, float (&dst)[ROWS][EB]) {
  for (int i = threadIdx.x; i < ROWS * EB; i += 256) {
    const int r = i / EB, e = i % EB;
    const bool live = s0 + r < S && e < E;
    const float v = dl[live ? (s0 + r) * ldl + e : 0];
    dst[r][e] = live ? v : 0.0f;
  }
  __syncthreads();
}

// dx[s][m] = sum_e dl[s][e] * w[e][m] (e ascending, fp32, rounded once).  A thread keeps its m-vector of every expert
// row in registers and walks the token rows of its workgroup's block; dl[s][*] comes from LDS.
template <typename T, int EB>
__global__ __launch_bounds__(256) void gate_dgrad_kernel(const float* dl, long ldl, const T* w, long ldw, long S, int M,
                                                         int E, T* dx, long ldx, const T* init, long ld_init) {
  constexpr int VEC = Vec16<T>::N;
  __shared__ float dls[kGateDgradRows][EB];
  const int c = blockIdx.x * 256 + threadIdx.x;
  const bool active = c < M / VEC;
  Vec16<T> wv[EB];
#pragma unroll
  for (int e = 0; e < EB; ++e) wv[e].q = *reinterpret_cast<const uint4*>(w + (e < E ? e : 0) * ldw + (active ? c : 0) * VEC);
  const long s0 = (long)blockIdx.y * kGateDgradRows;
  stage_dl<kGateDgradRows, EB>(dl, ldl, s0, S, E, dls);
  if (!active) return;
#pragma unroll 4
  for (int r = 0; r < kGateDgradRows; ++r) {
    if (s0 + r >= S) break;
    float o[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) o[k] = 0.0f;
#pragma unroll
    for (int e = 0; e < EB; ++e) {
      const float d = dls[r][e];  // zero for slots beyond E
#pragma unroll
      for (int k = 0; k < VEC; ++k) o[k] += d * to_f32(wv[e].e[k]);
    }
    Vec16<T> ov;
#pragma unroll
    for (int k = 0; k < VEC; ++k) ov.e[k] = from_f32<T>(o[k]);
    if (init != nullptr) {
      // the gradient that reached the same input along another path: added as autograd would add the two rounded
      // tensors (sum of the rounded values, rounded once more)
      Vec16<T> iv;
      iv.q = *reinterpret_cast<const uint4*>(init + (s0 + r) * ld_init + c * VEC);
#pragma unroll
      for (int k = 0; k < VEC; ++k) ov.e[k] = from_f32<T>(to_f32(iv.e[k]) + to_f32(ov.e[k]));
    }
    *reinterpret_cast<uint4*>(dx + (s0 + r) * ldx + c * VEC) = ov.q;
  }
}

// part[rb][e][m] = sum over the token rows s of block rb (ascending) of dl[s][e] * x[s][m]; 4 consecutive m per thread.
// Rows are taken kGateWgradBatch at a time with every load of a batch issued before the first use: the loop is a chain
// of memory round trips otherwise (one wavefront per SIMD, nothing else to switch to).
constexpr int kGateWgradBatch = 16;
template <typename T, int EB>
__global__ __launch_bounds__(256) void gate_wgrad_partial_kernel(const float* dl, long ldl, const T* x, long ldx, long S,
                                                                 int M, int E, float* part) {
  __shared__ float dls[kGateWgradRows][EB];
  const int c = blockIdx.x * 256 + threadIdx.x;  // group of 4 columns
  const bool active = c < M / 4;
  const long s0 = (long)blockIdx.y * kGateWgradRows;
  stage_dl<kGateWgradRows, EB>(dl, ldl, s0, S, E, dls);
  if (!active) return;
  union X4 {
    T e[4];
    uint2 u2;
    uint4 u4;
  };
  float acc[EB][4];
#pragma unroll
  for (int e = 0; e < EB; ++e)
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[e][k] = 0.0f;
  for (int b = 0; b < kGateWgradRows; b += kGateWgradBatch) {
    if (s0 + b >= S) break;
    X4 xv[kGateWgradBatch];
#pragma unroll
    for (int i = 0; i < kGateWgradBatch; ++i) {
      const long s = s0 + b + i < S ? s0 + b + i : S - 1;  // rows outside: re-read the last row, weighted by zero
      if (sizeof(T) == 2)
        xv[i].u2 = *reinterpret_cast<const uint2*>(x + s * ldx + c * 4);
      else
        xv[i].u4 = *reinterpret_cast<const uint4*>(x + s * ldx + c * 4);
    }
#pragma unroll
    for (int i = 0; i < kGateWgradBatch; ++i)
#pragma unroll
      for (int e = 0; e < EB; ++e) {
        const float d = dls[b + i][e];
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[e][k] += d * to_f32(xv[i].e[k]);
      }
  }
  float* out = part + (long)blockIdx.y * E * M;
#pragma unroll
  for (int e = 0; e < EB; ++e)
    if (e < E) *reinterpret_cast<float4*>(out + (long)e * M + c * 4) = make_float4(acc[e][0], acc[e][1], acc[e][2], acc[e][3]);
}

// dw[e][m..m+3] (+)= sum over the row blocks (ascending) of part[rb][e][m..m+3]; 16 partial vectors in flight per thread.
template <typename T>
__global__ __launch_bounds__(256) void gate_wgrad_final_kernel(const float* part, long nrb, int E, int M, T* dw,
                                                               long ld_dw, int accumulate) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)E * (M / 4)) return;
  const long e = idx / (M / 4), m = (idx - e * (M / 4)) * 4;
  const long stride = (long)E * M;
  const float* src = part + e * M + m;
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (long rb = 0; rb < nrb; rb += 16) {
    float4 v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = *reinterpret_cast<const float4*>(src + (rb + i < nrb ? rb + i : nrb - 1) * stride);
#pragma unroll
    for (int i = 0; i < 16; ++i)
      if (rb + i < nrb) acc[0] += v[i].x, acc[1] += v[i].y, acc[2] += v[i].z, acc[3] += v[i].w;
  }
  T* dst = dw + e * ld_dw + m;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float a = acc[k];
    if (accumulate) a += to_f32(dst[k]);
    dst[k] = from_f32<T>(a);
  }
}

static int gate_check(const char* who, int dtype, int64_t S, int64_t M, int64_t E) {
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "%s: unknown dtype %d", who, dtype);
  const int64_t vec = dtype == RTP_F32 ? 4 : 8;
  RTP_REQUIRE(S >= 1 && S < (1ll << 31), "%s: %lld token rows out of range", who, (long long)S);
  RTP_REQUIRE(E >= 1 && E <= kGateMaxExperts, "%s: %lld experts, at most %d", who, (long long)E, kGateMaxExperts);
  RTP_REQUIRE(M >= vec && M % vec == 0 && M < (1ll << 24), "%s: model dimension %lld must be a multiple of %lld", who,
              (long long)M, (long long)vec);
  return RTP_OK;
}
static bool aligned16(const void* p) { return (uintptr_t)p % 16 == 0; }

// KERNEL<T, EB> with the smallest EB in {4, 8, 16} that holds E
#define RTP_GATE_LAUNCH(KERNEL, T, E, GRID, ST, ...)                                          \
  do {                                                                                         \
    if ((E) <= 4)                                                                              \
      hipLaunchKernelGGL((KERNEL<T, 4>), GRID, dim3(256), 0, ST, __VA_ARGS__);                 \
    else if ((E) <= 8)                                                                         \
      hipLaunchKernelGGL((KERNEL<T, 8>), GRID, dim3(256), 0, ST, __VA_ARGS__);                 \
    else                                                                                       \
      hipLaunchKernelGGL((KERNEL<T, 16>), GRID, dim3(256), 0, ST, __VA_ARGS__);                \
  } while (0)

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_gate_supported(int dtype, int64_t experts, int64_t model_dim) {
  if (dtype != RTP_F32 && dtype != RTP_BF16) return 0;
  const int64_t vec = dtype == RTP_F32 ? 4 : 8;
  return experts >= 1 && experts <= kGateMaxExperts && model_dim >= vec && model_dim % vec == 0 && model_dim < (1ll << 24);
}

extern "C" int rtp_gate_fwd(void* stream, int dtype, const void* x, int64_t ldx, const void* w, int64_t ldw, int64_t S,
                            int64_t M, int64_t E, float* logits, int64_t ld_logits) {
  if (int rc = gate_check("rtp_gate_fwd", dtype, S, M, E)) return rc;
  const int64_t vec = dtype == RTP_F32 ? 4 : 8;
  RTP_REQUIRE(x && w && logits, "rtp_gate_fwd: null pointer");
  RTP_REQUIRE(aligned16(x) && aligned16(w) && ldx % vec == 0 && ldw % vec == 0 && ldx >= M && ldw >= M && ld_logits >= E,
              "rtp_gate_fwd: x and w must be 16-byte aligned with row pitches >= M that are multiples of %lld",
              (long long)vec);
  hipStream_t st = (hipStream_t)stream;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "gate_fwd", 2.0 * S * M * E, esz * ((double)S * M + (double)E * M) + 4.0 * S * E);
  const dim3 grid((unsigned)ceil_div(S, 4 * kGateFwdRows));
  if (dtype == RTP_F32)
    RTP_GATE_LAUNCH(gate_fwd_kernel, float, E, grid, st, (const float*)x, (long)ldx, (const float*)w, (long)ldw, (long)S,
                    (int)M, (int)E, logits, (long)ld_logits);
  else
    RTP_GATE_LAUNCH(gate_fwd_kernel, bf16_t, E, grid, st, (const bf16_t*)x, (long)ldx, (const bf16_t*)w, (long)ldw,
                    (long)S, (int)M, (int)E, logits, (long)ld_logits);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_gate_dgrad(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* w,
                              int64_t ldw, int64_t S, int64_t M, int64_t E, void* dx, int64_t ldx, const void* dx_init,
                              int64_t ld_dx_init) {
  if (int rc = gate_check("rtp_gate_dgrad", dtype, S, M, E)) return rc;
  const int64_t vec = dtype == RTP_F32 ? 4 : 8;
  RTP_REQUIRE(dlogits && w && dx, "rtp_gate_dgrad: null pointer");
  RTP_REQUIRE(aligned16(dx) && aligned16(w) && ldx % vec == 0 && ldw % vec == 0 && ldx >= M && ldw >= M &&
                  ld_dlogits >= E,
              "rtp_gate_dgrad: dx and w must be 16-byte aligned with row pitches >= M that are multiples of %lld",
              (long long)vec);
  RTP_REQUIRE(dx_init == nullptr || (aligned16(dx_init) && ld_dx_init % vec == 0 && ld_dx_init >= M),
              "rtp_gate_dgrad: dx_init must be 16-byte aligned with a row pitch >= M that is a multiple of %lld",
              (long long)vec);
  hipStream_t st = (hipStream_t)stream;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "gate_dgrad", 2.0 * S * M * E,
                    esz * ((double)S * M * (dx_init ? 2.0 : 1.0) + (double)E * M) + 4.0 * S * E);
  const dim3 grid((unsigned)ceil_div(M / vec, 256), (unsigned)ceil_div(S, kGateDgradRows));
  if (dtype == RTP_F32)
    RTP_GATE_LAUNCH(gate_dgrad_kernel, float, E, grid, st, dlogits, (long)ld_dlogits, (const float*)w, (long)ldw, (long)S,
                    (int)M, (int)E, (float*)dx, (long)ldx, (const float*)dx_init, (long)ld_dx_init);
  else
    RTP_GATE_LAUNCH(gate_dgrad_kernel, bf16_t, E, grid, st, dlogits, (long)ld_dlogits, (const bf16_t*)w, (long)ldw,
                    (long)S, (int)M, (int)E, (bf16_t*)dx, (long)ldx, (const bf16_t*)dx_init, (long)ld_dx_init);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" size_t rtp_gate_wgrad_workspace_bytes(int64_t S, int64_t M, int64_t E) {
  if (S < 1 || M < 1 || E < 1) return 0;
  return (size_t)ceil_div(S, kGateWgradRows) * (size_t)E * (size_t)M * sizeof(float);
}

// The two launches of the weight gradient; `part` holds ceil(S / 64) * E * M floats, every one of which the first
// kernel writes before the second reads it (nothing has to start at zero).
static int gate_wgrad_launch(hipStream_t st, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x,
                             int64_t ldx, int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw, int accumulate,
                             float* part) {
  const long nrb = ceil_div(S, kGateWgradRows);
  const dim3 grid((unsigned)ceil_div(M / 4, 256), (unsigned)nrb);
  const dim3 fgrid((unsigned)ceil_div(E * (M / 4), 256));
  if (dtype == RTP_F32) {
    RTP_GATE_LAUNCH(gate_wgrad_partial_kernel, float, E, grid, st, dlogits, (long)ld_dlogits, (const float*)x, (long)ldx,
                    (long)S, (int)M, (int)E, part);
    hipLaunchKernelGGL(gate_wgrad_final_kernel<float>, fgrid, dim3(256), 0, st, part, nrb, (int)E, (int)M, (float*)dw,
                       (long)ld_dw, accumulate);
  } else {
    RTP_GATE_LAUNCH(gate_wgrad_partial_kernel, bf16_t, E, grid, st, dlogits, (long)ld_dlogits, (const bf16_t*)x,
                    (long)ldx, (long)S, (int)M, (int)E, part);
    hipLaunchKernelGGL(gate_wgrad_final_kernel<bf16_t>, fgrid, dim3(256), 0, st, part, nrb, (int)E, (int)M, (bf16_t*)dw,
                       (long)ld_dw, accumulate);
  }
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

static int gate_wgrad_check(const char* who, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x,
                            int64_t ldx, int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw) {
  if (int rc = gate_check(who, dtype, S, M, E)) return rc;
  const int64_t vec = dtype == RTP_F32 ? 4 : 8;
  RTP_REQUIRE(dlogits && x && dw, "%s: null pointer", who);
  RTP_REQUIRE(aligned16(x) && ldx % vec == 0 && ldx >= M && ld_dw >= M && ld_dlogits >= E,
              "%s: x must be 16-byte aligned, row pitches >= M (x: a multiple of %lld)", who, (long long)vec);
  return RTP_OK;
}

extern "C" int rtp_gate_wgrad(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x,
                              int64_t ldx, int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw, int accumulate,
                              void* workspace, size_t workspace_bytes) {
  if (int rc = gate_wgrad_check("rtp_gate_wgrad", dtype, dlogits, ld_dlogits, x, ldx, S, M, E, dw, ld_dw)) return rc;
  RTP_REQUIRE(workspace && aligned16(workspace), "rtp_gate_wgrad: the workspace must be a 16-byte aligned pointer");
  RTP_REQUIRE(workspace_bytes >= rtp_gate_wgrad_workspace_bytes(S, M, E), "rtp_gate_wgrad: workspace of %zu bytes, need %zu",
              workspace_bytes, rtp_gate_wgrad_workspace_bytes(S, M, E));
  hipStream_t st = (hipStream_t)stream;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  const long nrb = ceil_div(S, kGateWgradRows);
  ProfileScope prof(st, "gate_wgrad", 2.0 * S * M * E, esz * ((double)S * M + (double)E * M) + 4.0 * S * E + 8.0 * nrb * E * M);
  return gate_wgrad_launch(st, dtype, dlogits, ld_dlogits, x, ldx, S, M, E, dw, ld_dw, accumulate, (float*)workspace);
}

// ---- the same weight gradient for callers that cannot allocate -------------------------------------------------
// The partial sums go to a buffer that is part of the library's code object instead of a caller's workspace.  In host
// code the array's name is only a stand-in for the symbol: the device address of each GPU's own copy is asked for
// once per device (with that device current) and kept; kernels and everything else only ever see that address.
namespace rtp {
constexpr size_t kGateStaticScratchBytes = RTP_GATE_WGRAD_STATIC_MAX_BYTES;
static __device__ __align__(256) unsigned char gate_wgrad_scratch[kGateStaticScratchBytes];

constexpr int kMaxDevices = 64;
static std::mutex gate_scratch_mutex;
static void* gate_scratch_ptr[kMaxDevices];  // per device, nullptr until resolved

static int gate_scratch_for_current_device(float** out) {
  int dev = -1;
  RTP_HIP_TRY(hipGetDevice(&dev));
  RTP_REQUIRE(dev >= 0 && dev < kMaxDevices, "rtp_gate_wgrad_static: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(gate_scratch_mutex);
  if (!gate_scratch_ptr[dev]) {
    void* p = nullptr;
    RTP_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(gate_wgrad_scratch)));
    RTP_REQUIRE(p != nullptr, "rtp_gate_wgrad_static: the scratch symbol has no address on device %d", dev);
    gate_scratch_ptr[dev] = p;
  }
  *out = (float*)gate_scratch_ptr[dev];
  return RTP_OK;
}

// Called by rtp_device_check (the library's per-device set-up call) so that the address is known before a caller's
// first rtp_gate_wgrad_static; that entry point resolves it itself on a device nobody checked.
int gate_static_setup() {
  float* p = nullptr;
  return gate_scratch_for_current_device(&p);
}

}  // namespace rtp

extern "C" int rtp_gate_wgrad_static(void* stream, int dtype, const float* dlogits, int64_t ld_dlogits, const void* x,
                                     int64_t ldx, int64_t S, int64_t M, int64_t E, void* dw, int64_t ld_dw,
                                     int accumulate) {
  if (int rc = gate_wgrad_check("rtp_gate_wgrad_static", dtype, dlogits, ld_dlogits, x, ldx, S, M, E, dw, ld_dw))
    return rc;
  const size_t need = rtp_gate_wgrad_workspace_bytes(S, M, E);
  RTP_REQUIRE(need <= kGateStaticScratchBytes,
              "rtp_gate_wgrad_static: ceil(S / 64) * E * M * 4 = %zu bytes of partial sums exceed the built-in %zu; use "
              "rtp_gate_wgrad with a workspace",
              need, kGateStaticScratchBytes);
  float* part = nullptr;
  if (int rc = gate_scratch_for_current_device(&part)) return rc;
  return gate_wgrad_launch((hipStream_t)stream, dtype, dlogits, ld_dlogits, x, ldx, S, M, E, dw, ld_dw, accumulate, part);
}
