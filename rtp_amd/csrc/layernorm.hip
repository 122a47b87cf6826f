// Residual add fused with LayerNorm, forward and backward, for the post-LN decoder layers
// (y = LayerNorm(x + r) * gamma + beta).  A workgroup of 256 threads owns a row (forward) or a block of 4 rows
// (backward); a thread owns the same 16-byte column vectors in every row, so the gamma / beta gradient of a
// column never leaves its thread.  fp32 statistics: cross-lane reduction, then the 4 wavefronts through LDS;
// mean first, then the variance around it.
#include "common.h"

namespace rtp {

constexpr int kLnThreads = 256;
constexpr int kLnMaxVectors = 4;   // 16-byte vectors per thread: rows of up to 8192 bf16 or 4096 fp32 columns
constexpr int kLnMaxCols = kLnMaxVectors * kLnThreads * 8;
constexpr int kLnBwdRows = 4;     // rows per workgroup in the backward

template <typename T>
struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  union {
    uint4 q;
    T e[N];
  };
};

// Sum of one value per thread over the workgroup, in a fixed order; `slot` is a [4] LDS array of its own.
__device__ __forceinline__ float block_sum(float v, float* slot) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) slot[threadIdx.x >> 6] = v;
  __syncthreads();
  return (slot[0] + slot[1]) + (slot[2] + slot[3]);
}

// z = x + r (rounded to T, as a separate elementwise add would), y = (z - mean) * rstd * gamma + beta.
template <typename T, int NV>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_fwd_kernel(const T* x, const T* r, const T* gamma,
                                                                       const T* beta, float eps, long rows, int cols,
                                                                       T* z_out, T* y, float* mean_out,
                                                                       float* rstd_out) {
  touch_kernel_arguments<88>();
  constexpr int VEC = Vec16<T>::N;
  __shared__ float slots[2][4];
  const long row = blockIdx.x;
  const int nvec = cols / VEC;
  float v[NV][VEC];
  Vec16<T> gm[NV], bt[NV];
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLnThreads;
    if (c < nvec) {
      Vec16<T> a, b;
      a.q = reinterpret_cast<const uint4*>(x + row * cols)[c];
      if (r) b.q = reinterpret_cast<const uint4*>(r + row * cols)[c];
      gm[i].q = reinterpret_cast<const uint4*>(gamma)[c];
      if (beta) bt[i].q = reinterpret_cast<const uint4*>(beta)[c];
      if (r) {
        Vec16<T> zz;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          zz.e[e] = from_f32<T>(to_f32(a.e[e]) + to_f32(b.e[e]));
          v[i][e] = to_f32(zz.e[e]);
        }
        if (z_out) reinterpret_cast<uint4*>(z_out + row * cols)[c] = zz.q;
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[i][e] = to_f32(a.e[e]);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum += v[i][e];
    }
  }
  const float mean = block_sum(sum, slots[0]) / (float)cols;
  float sq = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    if (threadIdx.x + i * kLnThreads < nvec) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = v[i][e] - mean;
        sq += d * d;
      }
    }
  }
  const float rstd = rsqrtf(block_sum(sq, slots[1]) / (float)cols + eps);
  if (threadIdx.x == 0) {
    mean_out[row] = mean;
    rstd_out[row] = rstd;
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLnThreads;
    if (c < nvec) {
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float t = (v[i][e] - mean) * rstd * to_f32(gm[i].e[e]);
        if (beta) t += to_f32(bt[i].e[e]);
        o.e[e] = from_f32<T>(t);
      }
      reinterpret_cast<uint4*>(y + row * cols)[c] = o.q;
    }
  }
}

// dz = rstd * (g - mean_c(g) - zhat * mean_c(g * zhat)),  g = dy * gamma,  zhat = (z - mean) * rstd.
// The gamma / beta gradient contributions of the workgroup's rows (dy * zhat, dy, added in row order) go to
// part[block][2][cols]; layernorm_bwd_final_kernel sums the blocks in a fixed order.
template <typename T, int NV>
__global__ __launch_bounds__(kLnThreads) void layernorm_bwd_kernel(const T* dy, const T* z, const T* gamma,
                                                                   const float* mean, const float* rstd, long rows,
                                                                   int cols, T* dz, float* part) {
  touch_kernel_arguments<72>();
  constexpr int VEC = Vec16<T>::N, RB = kLnBwdRows;
  __shared__ float slots[RB][2][4];
  const int nvec = cols / VEC;
  const long row0 = (long)blockIdx.x * RB;
  // Every load of the block is issued before the first reduction, and without branches (rows and vectors outside
  // re-read the block's first ones and are zeroed afterwards): a conditional load is a branch, and the compiler
  // waits for the loads of one row before it issues the next row's.
  Vec16<T> ra[RB][NV], rb[RB][NV], gm[NV];
  float mu[RB], rs[RB];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLnThreads;
    gm[i].q = reinterpret_cast<const uint4*>(gamma)[c < nvec ? c : 0];  // vectors outside meet zeroed dy / z only
  }
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    const bool live = row0 + rr < rows;
    const long r = live ? row0 + rr : row0;
    mu[rr] = mean[r];
    rs[rr] = rstd[r];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * kLnThreads;
      const int cc = c < nvec ? c : 0;
      ra[rr][i].q = reinterpret_cast<const uint4*>(dy + r * cols)[cc];
      rb[rr][i].q = reinterpret_cast<const uint4*>(z + r * cols)[cc];
    }
  }
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    const bool live = row0 + rr < rows;
    if (!live) mu[rr] = rs[rr] = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
      if (!live || threadIdx.x + i * kLnThreads >= nvec) {
        ra[rr][i].q = make_uint4(0u, 0u, 0u, 0u);
        rb[rr][i].q = make_uint4(0u, 0u, 0u, 0u);
      }
  }
  float dg[NV][VEC], db[NV][VEC];
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < VEC; ++e) dg[i][e] = db[i][e] = 0.0f;
  float s1[RB], s2[RB];
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    s1[rr] = s2[rr] = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float d = to_f32(ra[rr][i].e[e]);
        const float zh = (to_f32(rb[rr][i].e[e]) - mu[rr]) * rs[rr];  // 0 for rows / columns outside
        const float g = d * to_f32(gm[i].e[e]);
        s1[rr] += g;
        s2[rr] += g * zh;
        dg[i][e] += d * zh;
        db[i][e] += d;
      }
    s1[rr] = wave_sum(s1[rr]);
    s2[rr] = wave_sum(s2[rr]);
    if ((threadIdx.x & 63) == 0) {
      slots[rr][0][threadIdx.x >> 6] = s1[rr];
      slots[rr][1][threadIdx.x >> 6] = s2[rr];
    }
  }
  __syncthreads();
#pragma unroll
  for (int rr = 0; rr < RB; ++rr) {
    if (row0 + rr >= rows) break;
    const float m1 = ((slots[rr][0][0] + slots[rr][0][1]) + (slots[rr][0][2] + slots[rr][0][3])) / (float)cols;
    const float m2 = ((slots[rr][1][0] + slots[rr][1][1]) + (slots[rr][1][2] + slots[rr][1][3])) / (float)cols;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * kLnThreads;
      if (c < nvec) {
        Vec16<T> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float zh = (to_f32(rb[rr][i].e[e]) - mu[rr]) * rs[rr];
          const float g = to_f32(ra[rr][i].e[e]) * to_f32(gm[i].e[e]);
          o.e[e] = from_f32<T>(rs[rr] * (g - m1 - zh * m2));
        }
        reinterpret_cast<uint4*>(dz + (row0 + rr) * cols)[c] = o.q;
      }
    }
  }
  float* out = part + (long)blockIdx.x * 2 * cols;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * kLnThreads;
    if (c < nvec) {
#pragma unroll
      for (int e = 0; e < VEC; e += 4) {
        *reinterpret_cast<float4*>(out + c * VEC + e) = make_float4(dg[i][e], dg[i][e + 1], dg[i][e + 2], dg[i][e + 3]);
        *reinterpret_cast<float4*>(out + cols + c * VEC + e) =
            make_float4(db[i][e], db[i][e + 1], db[i][e + 2], db[i][e + 3]);
      }
    }
  }
}

// 32 columns of the [2][cols] sums per workgroup: 8 groups of threads each add an eighth of the blocks (a fixed
// order, sixteen loads in flight), then the eighths are added in order.
template <typename T>
__device__ __forceinline__ void ln_final_columns(const float* part, long nblocks, int cols, T* dgamma, T* dbeta) {
  __shared__ float eighth[8][32];
  const int cl = threadIdx.x & 31, grp = threadIdx.x >> 5;
  const int c = blockIdx.x * 32 + cl;  // column of the [2 * cols] row
  const long per = (nblocks + 7) / 8;
  const long b0 = grp * per, b1 = b0 + per < nblocks ? b0 + per : nblocks;
  float acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = 0.0f;
  if (c < 2 * cols) {
    long b = b0;
    for (; b + 15 < b1; b += 16) {
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] += part[(b + j) * 2 * cols + c];
    }
    for (; b < b1; ++b) acc[0] += part[b * 2 * cols + c];
  }
#pragma unroll
  for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
    for (int j = 0; j < w; ++j) acc[j] += acc[j + w];
  eighth[grp][cl] = acc[0];
  __syncthreads();
  if (grp == 0 && c < 2 * cols) {
    float s = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s += eighth[e][cl];
    if (c < cols) {
      dgamma[c] = from_f32<T>(s);
    } else if (dbeta) {
      dbeta[c - cols] = from_f32<T>(s);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void layernorm_bwd_final_kernel(const float* part, long nblocks, int cols, T* dgamma,
                                                                  T* dbeta) {
  ln_final_columns<T>(part, nblocks, cols, dgamma, dbeta);
}

// The same reduction for many LayerNorms in one launch: blockIdx.y picks the entry of a device-resident table.  Their
// parameter gradients are not needed before the backward pass ends, so one launch there replaces one per layer.
struct LnFinalItem {
  const float* part;
  long nblocks, cols;
  void *dgamma, *dbeta;
};
template <typename T>
__global__ __launch_bounds__(256) void layernorm_bwd_final_many_kernel(const LnFinalItem* items) {
  const LnFinalItem it = items[blockIdx.y];
  if ((long)blockIdx.x * 32 >= 2 * it.cols) return;  // the grid is sized for the widest entry
  ln_final_columns<T>(it.part, it.nblocks, (int)it.cols, (T*)it.dgamma, (T*)it.dbeta);
}

static int ln_nv(int dtype, int64_t cols) {
  const int vec = dtype == RTP_F32 ? 4 : 8;
  if (cols <= 0 || cols % vec || cols / vec > (int64_t)kLnMaxVectors * kLnThreads) return 0;
  const int nv = (int)ceil_div(cols / vec, kLnThreads);
  return nv == 3 ? 4 : nv;  // instantiated for 1, 2 and 4
}

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_layernorm_supported(int dtype, int64_t cols) {
  return (dtype == RTP_F32 || dtype == RTP_BF16) && ln_nv(dtype, cols) != 0;
}

#define RTP_LN_DISPATCH(KERNEL, T, NVV, ...)                          \
  if ((NVV) == 1) {                                                   \
    hipLaunchKernelGGL((KERNEL<T, 1>), __VA_ARGS__);                  \
  } else if ((NVV) == 2) {                                            \
    hipLaunchKernelGGL((KERNEL<T, 2>), __VA_ARGS__);                  \
  } else {                                                            \
    hipLaunchKernelGGL((KERNEL<T, 4>), __VA_ARGS__);                  \
  }

extern "C" int rtp_add_layernorm_fwd(void* stream, int dtype, const void* x, const void* r, const void* gamma,
                                     const void* beta, float eps, int64_t rows, int64_t cols, void* z_out, void* y,
                                     float* mean, float* rstd) {
  RTP_REQUIRE(x && gamma && y && mean && rstd, "rtp_add_layernorm_fwd: null pointer");
  RTP_REQUIRE(rows >= 0 && rows < (1ll << 31), "rtp_add_layernorm_fwd: row count %lld out of range", (long long)rows);
  const int nv = ln_nv(dtype, cols);
  RTP_REQUIRE((dtype == RTP_F32 || dtype == RTP_BF16) && nv,
              "rtp_add_layernorm_fwd: dtype %d with %lld columns is not supported (whole 16-byte vectors, at most %d of them)",
              dtype, (long long)cols, kLnMaxVectors * kLnThreads);
  RTP_REQUIRE(((uintptr_t)x | (uintptr_t)r | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)z_out | (uintptr_t)y) % 16 == 0,
              "rtp_add_layernorm_fwd: operands must be 16-byte aligned");
  if (rows == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "add_layernorm_fwd", 0.0, (double)rows * cols * esz * (2.0 + (r ? 1.0 : 0.0) + (r && z_out ? 1.0 : 0.0)));
  const dim3 grid((unsigned)rows), block(kLnThreads);
  if (dtype == RTP_F32) {
    RTP_LN_DISPATCH(add_layernorm_fwd_kernel, float, nv, grid, block, 0, st, (const float*)x, (const float*)r,
                    (const float*)gamma, (const float*)beta, eps, (long)rows, (int)cols, (float*)z_out, (float*)y, mean,
                    rstd)
  } else {
    RTP_LN_DISPATCH(add_layernorm_fwd_kernel, bf16_t, nv, grid, block, 0, st, (const bf16_t*)x, (const bf16_t*)r,
                    (const bf16_t*)gamma, (const bf16_t*)beta, eps, (long)rows, (int)cols, (bf16_t*)z_out, (bf16_t*)y,
                    mean, rstd)
  }
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" size_t rtp_layernorm_bwd_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 256;
  return (size_t)(ceil_div(rows, kLnBwdRows) * 2 * cols * 4 + 256);
}

extern "C" int rtp_layernorm_bwd(void* stream, int dtype, const void* dy, const void* z, const void* gamma,
                                 const float* mean, const float* rstd, int64_t rows, int64_t cols, void* dz,
                                 void* dgamma, void* dbeta, void* workspace, size_t workspace_bytes) {
  RTP_REQUIRE(dy && z && gamma && mean && rstd && dz && workspace, "rtp_layernorm_bwd: null pointer");
  RTP_REQUIRE(dgamma || !dbeta, "rtp_layernorm_bwd: dbeta without dgamma");
  RTP_REQUIRE(rows >= 1 && rows < (1ll << 31), "rtp_layernorm_bwd: row count %lld out of range", (long long)rows);
  const int nv = ln_nv(dtype, cols);
  RTP_REQUIRE((dtype == RTP_F32 || dtype == RTP_BF16) && nv,
              "rtp_layernorm_bwd: dtype %d with %lld columns is not supported", dtype, (long long)cols);
  RTP_REQUIRE(((uintptr_t)dy | (uintptr_t)z | (uintptr_t)gamma | (uintptr_t)dz) % 16 == 0,
              "rtp_layernorm_bwd: operands must be 16-byte aligned");
  const int64_t nblocks = ceil_div(rows, kLnBwdRows);
  if (workspace_bytes < (size_t)(nblocks * 2 * cols * 4))
    return fail(RTP_ERR_WORKSPACE, "rtp_layernorm_bwd: workspace %zu < required %lld", workspace_bytes,
                (long long)(nblocks * 2 * cols * 4));
  hipStream_t st = (hipStream_t)stream;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "layernorm_bwd", 0.0, (double)rows * cols * esz * 3.0);
  const dim3 grid((unsigned)nblocks), block(256);
  const size_t lds = 0;
  float* part = (float*)workspace;
  if (dtype == RTP_F32) {
    RTP_LN_DISPATCH(layernorm_bwd_kernel, float, nv, grid, block, lds, st, (const float*)dy, (const float*)z,
                    (const float*)gamma, mean, rstd, (long)rows, (int)cols, (float*)dz, part)
    if (dgamma)
      hipLaunchKernelGGL(layernorm_bwd_final_kernel<float>, dim3((unsigned)ceil_div(2 * cols, 32)), block, 0, st, part,
                         (long)nblocks, (int)cols, (float*)dgamma, (float*)dbeta);
  } else {
    RTP_LN_DISPATCH(layernorm_bwd_kernel, bf16_t, nv, grid, block, lds, st, (const bf16_t*)dy, (const bf16_t*)z,
                    (const bf16_t*)gamma, mean, rstd, (long)rows, (int)cols, (bf16_t*)dz, part)
    if (dgamma)
      hipLaunchKernelGGL(layernorm_bwd_final_kernel<bf16_t>, dim3((unsigned)ceil_div(2 * cols, 32)), block, 0, st, part,
                         (long)nblocks, (int)cols, (bf16_t*)dgamma, (bf16_t*)dbeta);
  }
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int64_t rtp_layernorm_bwd_blocks(int64_t rows) { return rows <= 0 ? 0 : ceil_div(rows, kLnBwdRows); }

extern "C" int rtp_layernorm_bwd_finalize(void* stream, int dtype, const rtp_ln_final_item* items, int64_t n_items,
                                          int64_t max_cols) {
  static_assert(sizeof(rtp_ln_final_item) == sizeof(LnFinalItem), "rtp_ln_final_item layout");
  RTP_REQUIRE(items, "rtp_layernorm_bwd_finalize: null table");
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_layernorm_bwd_finalize: unknown dtype %d", dtype);
  RTP_REQUIRE(n_items >= 0 && n_items < 65536, "rtp_layernorm_bwd_finalize: %lld entries out of range", (long long)n_items);
  RTP_REQUIRE(max_cols >= 1 && max_cols <= kLnMaxCols, "rtp_layernorm_bwd_finalize: widest entry %lld out of range",
              (long long)max_cols);
  if (n_items == 0) return RTP_OK;
  hipStream_t st = (hipStream_t)stream;
  ProfileScope prof(st, "layernorm_bwd_finalize", 0.0, 0.0);
  const dim3 grid((unsigned)ceil_div(2 * max_cols, 32), (unsigned)n_items);
  const LnFinalItem* table = reinterpret_cast<const LnFinalItem*>(items);
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(layernorm_bwd_final_many_kernel<float>, grid, dim3(256), 0, st, table);
  else
    hipLaunchKernelGGL(layernorm_bwd_final_many_kernel<bf16_t>, grid, dim3(256), 0, st, table);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
