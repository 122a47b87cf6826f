// Sharded embedding: coalesced row gather and a deterministic (sorted, segmented) scatter-add.
#include <cstring>

#include "common.h"

#include <rocprim/rocprim.hpp>

namespace rtp {

// One workgroup per (token, 4 KiB column chunk); 16-byte lanes when the shard rectangle allows it.
// With `pos` the row is scaled and a positional row added on the way: out = T(T(table * scale) + pos[t / batch]),
// each step rounded to T as the two separate element-wise operations would round it.
template <typename T>
__global__ __launch_bounds__(256) void gather_kernel(const T* table, long ld_table, long row_begin, long row_count,
                                                     long cols, const int64_t* ids, T* out, long ld_out, int vec,
                                                     long table_sg, long out_sg, float scale, const T* pos, long ld_pos,
                                                     long pos_sg, long batch) {
  const long t = blockIdx.x;
  const long row = ids[t] - row_begin;
  if (row < 0 || row >= row_count) return;
  const T* src = table + blockIdx.z * table_sg + row * ld_table;
  T* dst = out + blockIdx.z * out_sg + t * ld_out;
  constexpr int VEC = 16 / sizeof(T);
  if (pos) {
    const T* prow = pos + (long)((unsigned)t / (unsigned)batch) * ld_pos + blockIdx.z * pos_sg;
    if (vec) {
      const long nvec = cols / VEC;
      union Pack {
        uint4 u;
        T e[VEC];
      };
      for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < nvec; i += (long)gridDim.y * 256) {
#pragma clang fp contract(off)
        Pack a, b, r;
        a.u = reinterpret_cast<const uint4*>(src)[i];
        b.u = reinterpret_cast<const uint4*>(prow)[i];
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          r.e[e] = from_f32<T>(to_f32(from_f32<T>(to_f32(a.e[e]) * scale)) + to_f32(b.e[e]));
        reinterpret_cast<uint4*>(dst)[i] = r.u;
      }
      return;
    }
    for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < cols; i += (long)gridDim.y * 256) {
#pragma clang fp contract(off)
      const float a = to_f32(from_f32<T>(to_f32(src[i]) * scale));
      dst[i] = from_f32<T>(a + to_f32(prow[i]));
    }
    return;
  }
  if (vec) {
    const long nvec = cols / VEC;
    const uint4* s = reinterpret_cast<const uint4*>(src);
    uint4* d = reinterpret_cast<uint4*>(dst);
    for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < nvec; i += (long)gridDim.y * 256) d[i] = s[i];
  } else {
    for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < cols; i += (long)gridDim.y * 256) dst[i] = src[i];
  }
}

__global__ __launch_bounds__(256) void sort_prep_kernel(const int64_t* ids, long n, int* keys, int* vals) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) {
    keys[i] = (int)ids[i];
    vals[i] = (int)i;
  }
}

// (id, position) pairs of up to kSortLdsMax token ids sorted by one workgroup in LDS: a bitonic network over the
// 64-bit words id << 32 | position (all different, so the order is total and the result is the stable sort by id).
// A step's 1024 ids take 55 compare-exchange rounds of a few hundred nanoseconds each; a device-wide radix sort
// spends several launches on them.  Slots beyond n hold the largest word and stay at the end.
constexpr int kSortLdsMax = 8192;  // 64 KiB of LDS
constexpr int kSortThreads = 1024;
__global__ __launch_bounds__(kSortThreads) void sort_ids_lds_kernel(const int64_t* ids, int n, int npow2, int* keys,
                                                                    int* vals) {
  extern __shared__ unsigned long long sort_words[];
  for (int i = threadIdx.x; i < npow2; i += kSortThreads)
    sort_words[i] = i < n ? ((unsigned long long)(unsigned)(int)ids[i] << 32) | (unsigned)i : ~0ull;
  __syncthreads();
  for (int k = 2; k <= npow2; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < (npow2 >> 1); t += kSortThreads) {
        const int lo = ((t & ~(j - 1)) << 1) | (t & (j - 1)), hi = lo | j;
        const unsigned long long a = sort_words[lo], b = sort_words[hi];
        const bool ascending = (lo & k) == 0;
        if ((a > b) == ascending) {
          sort_words[lo] = b;
          sort_words[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  for (int i = threadIdx.x; i < n; i += kSortThreads) {
    const unsigned long long w = sort_words[i];
    keys[i] = (int)(unsigned)(w >> 32);
    vals[i] = (int)(unsigned)(w & 0xffffffffull);
  }
}

__global__ __launch_bounds__(256) void zero_rows_kernel(char* base, long ld_bytes, long row_bytes, long rows,
                                                        long group_bytes) {
  const long r = blockIdx.x;
  if (r >= rows) return;
  char* p = base + blockIdx.z * group_bytes + r * ld_bytes;
  if ((((uintptr_t)p | (uintptr_t)row_bytes) & 15) == 0) {
    uint4* d = reinterpret_cast<uint4*>(p);
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < (row_bytes >> 4); i += (long)gridDim.y * 256) d[i] = z;
  } else {
    for (long i = (long)blockIdx.y * 256 + threadIdx.x; i < row_bytes; i += (long)gridDim.y * 256) p[i] = 0;
  }
}

// keys: token ids sorted ascending (stable), vals: their positions.  The workgroup at sorted index i
// owns the segment that starts there (if one does) and sums it front to back, i.e. in ascending
// position order, starting from +0.0f exactly like a sequential index_add_ into a zeroed table.
template <typename T, typename G>
__global__ __launch_bounds__(256) void scatter_kernel(const T* grad_out, long ld_go, long n, const int* keys,
                                                      const int* vals, G* grad_table, long ld_gt, long row_begin,
                                                      long row_count, long cols, long padding_idx, int scale_by_freq,
                                                      int overwrite, long go_sg, long gt_sg, float grad_scale,
                                                      float* master, T* weights, float lr, float clip, int store_grad) {
  grad_out += blockIdx.z * go_sg;  // group = shard: its column block of the upstream gradient, its own table
  grad_table += blockIdx.z * gt_sg;
  if (master != nullptr) master += blockIdx.z * gt_sg;
  if (weights != nullptr) weights += blockIdx.z * gt_sg;
  const long i = blockIdx.x;
  const int id = keys[i];
  if (i > 0 && keys[i - 1] == id) return;
  if (id == padding_idx) return;
  const long row = (long)id - row_begin;
  if (row < 0 || row >= row_count) return;
  long end = i + 1;
  while (end < n && keys[end] == id) ++end;
  const float inv = scale_by_freq ? 1.0f / (float)(end - i) : 1.0f;
  for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < cols; c += (long)gridDim.y * 256) {
    float acc = 0.0f;
    if (grad_scale == 1.0f) {
      for (long j = i; j < end; ++j) acc += to_f32(grad_out[(long)vals[j] * ld_go + c]);
    } else {
#pragma clang fp contract(off)
      // the upstream gradient of a scaled embedding: T(grad * scale), rounded as the separate multiplication would
      // (no fused multiply-add: the product is rounded before it joins the sum)
      for (long j = i; j < end; ++j)
        acc += to_f32(from_f32<T>(to_f32(grad_out[(long)vals[j] * ld_go + c]) * grad_scale));
    }
    if (scale_by_freq) acc *= inv;
    G* dst = grad_table + row * ld_gt + c;
    if (master != nullptr) {
      // clip + SGD applied where the row's gradient is produced (the caller guarantees that this is the row's whole
      // gradient of the step): the arithmetic of the separate update on the gradient as its table would hold it.
      // Rows no token names keep a zero gradient, which the update leaves alone, so they are not touched at all.
      const float w = sgd_update<G>(master[row * ld_gt + c], acc, lr, clip);
      master[row * ld_gt + c] = w;
      if (weights != nullptr) weights[row * ld_gt + c] = from_f32<T>(w);
      if (store_grad) *dst = from_f32<G>(acc);
      continue;
    }
    if (!overwrite) acc = to_f32(*dst) + acc;
    *dst = from_f32<G>(acc);
  }
}

// V consecutive elements of type X as floats and back; V > 1 means whole 16-byte vectors (the caller checked alignment).
template <typename X, int V>
__device__ __forceinline__ void vec_load(const X* p, float (&f)[V]) {
  if constexpr (V == 1) {
    f[0] = to_f32(p[0]);
  } else {
    constexpr int NQ = V * (int)sizeof(X) / 16;
    union {
      uint4 q[NQ];
      X e[V];
    } u;
#pragma unroll
    for (int q = 0; q < NQ; ++q) u.q[q] = reinterpret_cast<const uint4*>(p)[q];
#pragma unroll
    for (int v = 0; v < V; ++v) f[v] = to_f32(u.e[v]);
  }
}
template <typename X, int V>
__device__ __forceinline__ void vec_store(X* p, const float (&f)[V]) {
  if constexpr (V == 1) {
    p[0] = from_f32<X>(f[0]);
  } else {
    constexpr int NQ = V * (int)sizeof(X) / 16;
    union {
      uint4 q[NQ];
      X e[V];
    } u;
#pragma unroll
    for (int v = 0; v < V; ++v) u.e[v] = from_f32<X>(f[v]);
#pragma unroll
    for (int q = 0; q < NQ; ++q) reinterpret_cast<uint4*>(p)[q] = u.q[q];
  }
}

// The whole backward of the sharded embedding in ONE launch, for steps of up to kBwdMaxIds tokens: no sort.  Every
// workgroup stages the step's ids in LDS.  Workgroup t < n owns token position t: if an earlier position names the
// same id it leaves at once; otherwise it marks the later positions with that id in an LDS bitmap, lists them in
// ascending order and sums their upstream rows front to back, starting from +0.0f with position t -- the order of a
// sequential index_add_ into a zeroed table, for all shards (groups) of the layer.  With a zero fill requested the
// grid has further workgroups, one per block of table rows: each finds the rows of its block that no token names
// (bitmap over the same ids) and clears them; rows that are named are written in full by their token workgroup, so
// nothing is written twice and no ordering between the two kinds of workgroup is needed.
constexpr int kBwdMaxIds = 4096;
template <typename T, typename G, int V>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const T* grad_out, long ld_go, int n, const int64_t* ids,
                                                            G* grad_table, long ld_gt, long row_begin, long row_count,
                                                            long cols, long padding_idx, int scale_by_freq,
                                                            int overwrite, int groups, long go_sg, long gt_sg,
                                                            float grad_scale, float* master, T* weights, float lr,
                                                            float clip, int store_grad, int zero_rows) {
  __shared__ int s_ids[kBwdMaxIds];
  __shared__ unsigned s_bits[kBwdMaxIds / 32];
  __shared__ int s_count;
  const int tid = threadIdx.x;
  for (int i = tid; i < n; i += 256) s_ids[i] = (int)ids[i];
  for (int i = tid; i < kBwdMaxIds / 32; i += 256) s_bits[i] = 0u;
  __syncthreads();
  if ((long)blockIdx.x >= n) {
    // ---- rows that no token names: cleared ----
    const long r0 = ((long)blockIdx.x - n) * zero_rows;
    for (int i = tid; i < n; i += 256) {
      const int id = s_ids[i];
      const long r = (long)id - row_begin - r0;
      if (id != padding_idx && r >= 0 && r < zero_rows) atomicOr(&s_bits[r >> 5], 1u << (r & 31));
    }
    __syncthreads();
    const long per_row = cols / V;  // vectors of a row in one group
    const long total = (long)zero_rows * groups * per_row;
    for (long e = tid; e < total; e += 256) {
      const long r = e / (groups * per_row), rem = e - r * (groups * per_row);
      const long g = rem / per_row, c = (rem - g * per_row) * V;
      if (r0 + r >= row_count || ((s_bits[r >> 5] >> (r & 31)) & 1u)) continue;
      G* dst = grad_table + g * gt_sg + (r0 + r) * ld_gt + c;
      if (V == 1) {
        dst[0] = from_f32<G>(0.0f);
      } else {
        constexpr int NQ = V * (int)sizeof(G) / 16;
#pragma unroll
        for (int q = 0; q < NQ; ++q) reinterpret_cast<uint4*>(dst)[q] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
    return;
  }
  // ---- token position t ----
  const int t = blockIdx.x;
  const int id = s_ids[t];
  const long row = (long)id - row_begin;
  if (id == padding_idx || row < 0 || row >= row_count) return;
  int early = 0;
  for (int j = tid; j < t; j += 256) early |= (s_ids[j] == id) ? 1 : 0;
  if (__syncthreads_or(early)) return;  // an earlier position owns this id
  for (int j = t + tid; j < n; j += 256)
    if (s_ids[j] == id) atomicOr(&s_bits[j >> 5], 1u << (j & 31));
  __syncthreads();
  if (tid == 0) {
    // the positions with this id, ascending, written over the ids (which nobody reads any more)
    int cnt = 0;
    for (int w = t >> 5; w < (n + 31) / 32; ++w) {
      unsigned bits = s_bits[w];
      while (bits) {
        const int b = __builtin_ctz(bits);
        bits &= bits - 1;
        s_ids[cnt++] = w * 32 + b;
      }
    }
    s_count = cnt;
  }
  __syncthreads();
  const int cnt = s_count;
  const float inv = scale_by_freq ? 1.0f / (float)cnt : 1.0f;
  const long per_row = cols / V;
  for (long e = tid; e < (long)groups * per_row; e += 256) {
    const long g = e / per_row, c = (e - g * per_row) * V;
    const T* src = grad_out + g * go_sg + c;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = 0.0f;
    for (int k = 0; k < cnt; ++k) {
#pragma clang fp contract(off)
      const T* sp = src + (long)s_ids[k] * ld_go;
      union {
        uint4 q;
        T e[16 / sizeof(T)];
      } u;
      if (V == 1)
        u.e[0] = sp[0];
      else
        u.q = *reinterpret_cast<const uint4*>(sp);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        // grad_scale != 1: the upstream gradient of a scaled embedding, T(grad * scale), rounded as the separate
        // multiplication would round it before it joins the sum (no fused multiply-add)
        const float x = grad_scale == 1.0f ? to_f32(u.e[v]) : to_f32(from_f32<T>(to_f32(u.e[v]) * grad_scale));
        acc[v] += x;
      }
    }
    const long off = g * gt_sg + row * ld_gt + c;
    {
#pragma clang fp contract(off)
      if (scale_by_freq) {
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] *= inv;
      }
      if (master != nullptr) {
        // clip + SGD where the row's gradient is produced (the caller guarantees it is the row's whole gradient)
        float w[V];
        vec_load<float, V>(master + off, w);
#pragma unroll
        for (int v = 0; v < V; ++v) w[v] = sgd_update<G>(w[v], acc[v], lr, clip);
        vec_store<float, V>(master + off, w);
        if (weights != nullptr) vec_store<T, V>(weights + off, w);
        if (store_grad) vec_store<G, V>(grad_table + off, acc);
        continue;
      }
      if (!overwrite) {
        float old[V];
        vec_load<G, V>(grad_table + off, old);
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = old[v] + acc[v];
      }
      vec_store<G, V>(grad_table + off, acc);
    }
  }
}

struct SortLayout {
  size_t keys_in, vals_in, keys_out, vals_out, temp, total, temp_bytes;
};

static SortLayout sort_layout(int64_t n) {
  SortLayout L;
  const size_t arr = ((size_t)n * 4 + 255) & ~(size_t)255;
  L.keys_in = 0;
  L.vals_in = arr;
  L.keys_out = 2 * arr;
  L.vals_out = 3 * arr;
  L.temp = 4 * arr;
  size_t tb = 0;
  (void)rocprim::radix_sort_pairs(nullptr, tb, (const int*)nullptr, (int*)nullptr, (const int*)nullptr, (int*)nullptr,
                                  (unsigned)n, 0, 32, (hipStream_t) nullptr);
  L.temp_bytes = tb;
  L.total = L.temp + ((tb + 255) & ~(size_t)255) + 256;
  return L;
}

}  // namespace rtp

using namespace rtp;

static int gather_impl(void* stream, int dtype, const void* table, int64_t ld_table, int64_t row_begin,
                       int64_t row_count, int64_t cols, const int64_t* ids, int64_t n_ids, void* out, int64_t ld_out,
                       int64_t groups, int64_t table_sg, int64_t out_sg, float scale, const void* pos, int64_t ld_pos,
                       int64_t pos_sg, int64_t batch) {
  RTP_REQUIRE(table && ids && out, "rtp_embedding_gather: null pointer");
  RTP_REQUIRE(cols >= 0 && ld_table >= cols && ld_out >= cols && row_count >= 0 && n_ids >= 0,
              "rtp_embedding_gather: bad shape cols=%lld ld_table=%lld ld_out=%lld", (long long)cols,
              (long long)ld_table, (long long)ld_out);
  if (n_ids == 0 || cols == 0) return RTP_OK;
  RTP_REQUIRE(n_ids < (1ll << 31), "rtp_embedding_gather: too many ids");
  RTP_REQUIRE(groups >= 1 && groups < 65536, "rtp_embedding_gather: groups=%lld out of range", (long long)groups);
  const size_t esz = dtype == RTP_F32 ? 4 : 2;
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_embedding_gather: unknown dtype %d", dtype);
  const int vec = ((uintptr_t)table % 16 == 0) && ((uintptr_t)out % 16 == 0) && (ld_table * esz) % 16 == 0 &&
                  (ld_out * esz) % 16 == 0 && (cols * esz) % 16 == 0 && (table_sg * esz) % 16 == 0 &&
                  (out_sg * esz) % 16 == 0 &&
                  (!pos || ((uintptr_t)pos % 16 == 0 && (ld_pos * esz) % 16 == 0 && (pos_sg * esz) % 16 == 0));
  const unsigned chunks = (unsigned)std::min<int64_t>(16, std::max<int64_t>(1, ceil_div(cols * (int64_t)esz, 4096)));
  dim3 grid((unsigned)n_ids, chunks, (unsigned)groups);
  hipStream_t s = (hipStream_t)stream;
  ProfileScope prof(s, "embedding_gather", 0.0, (2.0 * (double)n_ids * cols * esz + 8.0 * n_ids) * groups);
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(gather_kernel<float>, grid, dim3(256), 0, s, (const float*)table, (long)ld_table,
                       (long)row_begin, (long)row_count, (long)cols, ids, (float*)out, (long)ld_out, vec,
                       (long)table_sg, (long)out_sg, scale, (const float*)pos, (long)ld_pos, (long)pos_sg,
                       (long)batch);
  else
    hipLaunchKernelGGL(gather_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)table, (long)ld_table,
                       (long)row_begin, (long)row_count, (long)cols, ids, (bf16_t*)out, (long)ld_out, vec,
                       (long)table_sg, (long)out_sg, scale, (const bf16_t*)pos, (long)ld_pos, (long)pos_sg,
                       (long)batch);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_embedding_gather(void* stream, int dtype, const void* table, int64_t ld_table, int64_t row_begin,
                                    int64_t row_count, int64_t cols, const int64_t* ids, int64_t n_ids, void* out,
                                    int64_t ld_out, int64_t groups, int64_t table_sg, int64_t out_sg) {
  return gather_impl(stream, dtype, table, ld_table, row_begin, row_count, cols, ids, n_ids, out, ld_out, groups,
                     table_sg, out_sg, 1.0f, nullptr, 0, 0, 1);
}

extern "C" int rtp_embedding_gather_scale_pos(void* stream, int dtype, const void* table, int64_t ld_table,
                                              int64_t row_begin, int64_t row_count, int64_t cols, const int64_t* ids,
                                              int64_t n_ids, void* out, int64_t ld_out, int64_t groups,
                                              int64_t table_sg, int64_t out_sg, float scale, const void* pos,
                                              int64_t ld_pos, int64_t pos_sg, int64_t batch) {
  RTP_REQUIRE(pos && batch >= 1 && batch < (1ll << 31) && ld_pos >= cols,
              "rtp_embedding_gather_scale_pos: need a positional table and 1 <= batch < 2^31");
  return gather_impl(stream, dtype, table, ld_table, row_begin, row_count, cols, ids, n_ids, out, ld_out, groups,
                     table_sg, out_sg, scale, pos, ld_pos, pos_sg, batch);
}

extern "C" size_t rtp_embedding_scatter_workspace_bytes(int64_t n_ids) {
  if (n_ids <= 0) return 256;
  return sort_layout(n_ids).total;
}

extern "C" int rtp_embedding_sort_ids(void* stream, const int64_t* ids, int64_t n_ids, void* workspace,
                                      size_t workspace_bytes) {
  RTP_REQUIRE(ids && workspace, "rtp_embedding_sort_ids: null pointer");
  RTP_REQUIRE(n_ids >= 0 && n_ids < (1ll << 31), "rtp_embedding_sort_ids: bad n_ids %lld", (long long)n_ids);
  if (n_ids == 0) return RTP_OK;
  RTP_REQUIRE((uintptr_t)workspace % 256 == 0, "rtp_embedding_sort_ids: workspace must be 256-byte aligned");
  const SortLayout L = sort_layout(n_ids);
  if (workspace_bytes < L.total)
    return fail(RTP_ERR_WORKSPACE, "rtp_embedding_sort_ids: workspace %zu < required %zu", workspace_bytes, L.total);
  char* w = (char*)workspace;
  hipStream_t s = (hipStream_t)stream;
  if (n_ids <= kSortLdsMax) {
    int npow2 = 2;
    while (npow2 < n_ids) npow2 <<= 1;
    ProfileScope prof(s, "embedding_sort_ids", 0.0, 16.0 * (double)n_ids);
    hipLaunchKernelGGL(sort_ids_lds_kernel, dim3(1), dim3(kSortThreads), (size_t)npow2 * 8, s, ids, (int)n_ids, npow2,
                       (int*)(w + L.keys_out), (int*)(w + L.vals_out));
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  }
  // more ids than one workgroup's LDS holds: the device-wide radix sort of rocPRIM
  hipLaunchKernelGGL(sort_prep_kernel, dim3((unsigned)ceil_div(n_ids, 256)), dim3(256), 0, s, ids, (long)n_ids,
                     (int*)(w + L.keys_in), (int*)(w + L.vals_in));
  RTP_LAUNCH_CHECK();
  size_t tb = L.temp_bytes;
  RTP_HIP_TRY(rocprim::radix_sort_pairs((void*)(w + L.temp), tb, (const int*)(w + L.keys_in), (int*)(w + L.keys_out),
                                        (const int*)(w + L.vals_in), (int*)(w + L.vals_out), (unsigned)n_ids, 0, 32,
                                        s));
  return RTP_OK;
}

static int scatter_impl(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out, int64_t n_ids,
                        const void* workspace, void* grad_table, int64_t ld_grad_table, int grad_table_f32,
                        int64_t row_begin, int64_t row_count, int64_t cols, int64_t padding_idx, int scale_by_freq,
                        int zero_fill, int64_t groups, int64_t grad_out_sg, int64_t grad_table_sg, float grad_scale,
                        float* master = nullptr, void* weights = nullptr, float lr = 0.0f, float clip = 0.0f,
                        int store_grad = 1) {
  RTP_REQUIRE(grad_out && workspace && grad_table, "rtp_embedding_scatter_add_det: null pointer");
  if (master != nullptr) {
    // the fused update replaces the dense gradient: nothing to fill unless the gradient is wanted as well
    RTP_REQUIRE(!grad_table_f32 || dtype == RTP_F32, "rtp_embedding_scatter_add_sgd: the gradient table has the table's dtype");
    RTP_REQUIRE(zero_fill || !store_grad, "rtp_embedding_scatter_add_sgd: a stored gradient starts from a zero fill");
    if (!store_grad) zero_fill = 0;
  }
  RTP_REQUIRE(groups >= 1 && groups < 65536, "rtp_embedding_scatter_add_det: groups %lld not in 1..65535",
              (long long)groups);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_embedding_scatter_add_det: unknown dtype %d", dtype);
  RTP_REQUIRE(cols >= 0 && ld_grad_out >= cols && ld_grad_table >= cols && row_count >= 0 && n_ids >= 0 &&
                  n_ids < (1ll << 31),
              "rtp_embedding_scatter_add_det: bad shape");
  if (cols == 0 || row_count == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t gsz = (dtype == RTP_F32 || grad_table_f32) ? 4 : 2;
  const unsigned chunks = (unsigned)std::min<int64_t>(16, std::max<int64_t>(1, ceil_div(cols, 1024)));
  if (zero_fill) {
    RTP_REQUIRE(row_count < (1ll << 31), "rtp_embedding_scatter_add_det: too many rows");
    ProfileScope prof(s, "embedding_grad_zero_fill", 0.0, (double)groups * row_count * cols * gsz);
    if (ld_grad_table == cols) {
      // a group's table is one contiguous block: fill it as such (a workgroup per 512-byte row slice is mostly idle)
      const int64_t bytes = row_count * cols * gsz;
      const unsigned wgs = (unsigned)std::min<int64_t>(2048, std::max<int64_t>(1, ceil_div(bytes, 16384)));
      hipLaunchKernelGGL(zero_rows_kernel, dim3(1, wgs, (unsigned)groups), dim3(256), 0, s, (char*)grad_table,
                         (long)bytes, (long)bytes, 1l, (long)(grad_table_sg * gsz));
    } else {
      hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)row_count, chunks, (unsigned)groups), dim3(256), 0, s,
                         (char*)grad_table, (long)(ld_grad_table * gsz), (long)(cols * gsz), (long)row_count,
                         (long)(grad_table_sg * gsz));
    }
    RTP_LAUNCH_CHECK();
  }
  if (n_ids == 0) return RTP_OK;
  const SortLayout L = sort_layout(n_ids);
  const char* w = (const char*)workspace;
  const int* keys = (const int*)(w + L.keys_out);
  const int* vals = (const int*)(w + L.vals_out);
  dim3 grid((unsigned)n_ids, chunks, (unsigned)groups);
  // After a zero fill the rows can simply be overwritten; otherwise the sum is added to what is there.
  const int overwrite = zero_fill ? 1 : 0;
#define RTP_SCATTER(T, G)                                                                                         \
  hipLaunchKernelGGL((scatter_kernel<T, G>), grid, dim3(256), 0, s, (const T*)grad_out, (long)ld_grad_out,         \
                     (long)n_ids, keys, vals, (G*)grad_table, (long)ld_grad_table, (long)row_begin, (long)row_count, \
                     (long)cols, (long)padding_idx, scale_by_freq, overwrite, (long)grad_out_sg, (long)grad_table_sg,  \
                     grad_scale, master, (T*)weights, lr, clip, store_grad)
  // algorithmic bytes: read every upstream row once, write (or read-modify-write) every touched row once
  ProfileScope prof(s, "embedding_scatter_add", (double)groups * n_ids * cols,
                    (double)groups * n_ids * cols * ((dtype == RTP_F32 ? 4.0 : 2.0) + (zero_fill ? 1.0 : 2.0) * gsz) + 8.0 * n_ids);
  if (dtype == RTP_F32)
    RTP_SCATTER(float, float);
  else if (grad_table_f32)
    RTP_SCATTER(bf16_t, float);
  else
    RTP_SCATTER(bf16_t, bf16_t);
#undef RTP_SCATTER
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_embedding_scatter_add_det(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out,
                                             int64_t n_ids, const void* workspace, void* grad_table,
                                             int64_t ld_grad_table, int grad_table_f32, int64_t row_begin,
                                             int64_t row_count, int64_t cols, int64_t padding_idx, int scale_by_freq,
                                             int zero_fill, int64_t groups, int64_t grad_out_sg,
                                             int64_t grad_table_sg) {
  return scatter_impl(stream, dtype, grad_out, ld_grad_out, n_ids, workspace, grad_table, ld_grad_table, grad_table_f32,
                      row_begin, row_count, cols, padding_idx, scale_by_freq, zero_fill, groups, grad_out_sg,
                      grad_table_sg, 1.0f);
}

extern "C" int rtp_embedding_scatter_add_scaled(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out,
                                                int64_t n_ids, const void* workspace, void* grad_table,
                                                int64_t ld_grad_table, int grad_table_f32, int64_t row_begin,
                                                int64_t row_count, int64_t cols, int64_t padding_idx,
                                                int scale_by_freq, int zero_fill, int64_t groups, int64_t grad_out_sg,
                                                int64_t grad_table_sg, float grad_scale) {
  return scatter_impl(stream, dtype, grad_out, ld_grad_out, n_ids, workspace, grad_table, ld_grad_table, grad_table_f32,
                      row_begin, row_count, cols, padding_idx, scale_by_freq, zero_fill, groups, grad_out_sg,
                      grad_table_sg, grad_scale);
}

extern "C" int rtp_embedding_scatter_add_sgd(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out,
                                             int64_t n_ids, const void* workspace, void* grad_table,
                                             int64_t ld_grad_table, int64_t row_begin, int64_t row_count, int64_t cols,
                                             int64_t padding_idx, int scale_by_freq, int64_t groups,
                                             int64_t grad_out_sg, int64_t grad_table_sg, float grad_scale,
                                             float* master, void* weights, float lr, float clip, int store_grad) {
  RTP_REQUIRE(master != nullptr, "rtp_embedding_scatter_add_sgd: null master");
  RTP_REQUIRE(dtype == RTP_F32 ? weights == nullptr || weights == (void*)master : true,
              "rtp_embedding_scatter_add_sgd: fp32 tables are their own master");
  return scatter_impl(stream, dtype, grad_out, ld_grad_out, n_ids, workspace, grad_table, ld_grad_table, 0, row_begin,
                      row_count, cols, padding_idx, scale_by_freq, store_grad ? 1 : 0, groups, grad_out_sg,
                      grad_table_sg, grad_scale, master, dtype == RTP_F32 ? nullptr : weights, lr, clip, store_grad);
}

extern "C" int rtp_embedding_backward_supported(int64_t n_ids) { return n_ids >= 0 && n_ids <= kBwdMaxIds ? 1 : 0; }

extern "C" int rtp_embedding_backward(void* stream, int dtype, const void* grad_out, int64_t ld_grad_out, int64_t n_ids,
                                      const int64_t* ids, void* grad_table, int64_t ld_grad_table, int grad_table_f32,
                                      int64_t row_begin, int64_t row_count, int64_t cols, int64_t padding_idx,
                                      int scale_by_freq, int zero_fill, int64_t groups, int64_t grad_out_sg,
                                      int64_t grad_table_sg, float grad_scale, float* master, void* weights, float lr,
                                      float clip, int store_grad) {
  RTP_REQUIRE(grad_out && grad_table && (ids || n_ids == 0), "rtp_embedding_backward: null pointer");
  RTP_REQUIRE(rtp_embedding_backward_supported(n_ids), "rtp_embedding_backward: %lld ids, at most %d (sort + scatter beyond)",
              (long long)n_ids, kBwdMaxIds);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_embedding_backward: unknown dtype %d", dtype);
  RTP_REQUIRE(groups >= 1 && groups < 65536, "rtp_embedding_backward: groups %lld not in 1..65535", (long long)groups);
  RTP_REQUIRE(cols >= 0 && ld_grad_out >= cols && ld_grad_table >= cols && row_count >= 0 && row_count < (1ll << 31),
              "rtp_embedding_backward: bad shape");
  if (master != nullptr) {
    RTP_REQUIRE(!grad_table_f32 || dtype == RTP_F32, "rtp_embedding_backward: with an update the gradient table has the table's dtype");
    RTP_REQUIRE(dtype != RTP_F32 || weights == nullptr || weights == (void*)master,
                "rtp_embedding_backward: fp32 tables are their own master");
    RTP_REQUIRE(zero_fill || !store_grad, "rtp_embedding_backward: a stored gradient beside the update starts from a zero fill");
    if (!store_grad) zero_fill = 0;  // the update replaces the dense gradient: nothing to fill
    if (dtype == RTP_F32) weights = nullptr;
  } else {
    store_grad = 1;
  }
  if (cols == 0 || row_count == 0 || (n_ids == 0 && !zero_fill)) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  const size_t esz = dtype == RTP_F32 ? 4 : 2, gsz = (dtype == RTP_F32 || grad_table_f32) ? 4 : 2;
  // 16-byte accesses when every row of every operand allows them
  const int64_t vec = 16 / (int64_t)esz;
  const bool aligned = cols % vec == 0 && (uintptr_t)grad_out % 16 == 0 && (ld_grad_out * esz) % 16 == 0 &&
                       (grad_out_sg * esz) % 16 == 0 && (uintptr_t)grad_table % 16 == 0 &&
                       (ld_grad_table * gsz) % 16 == 0 && (grad_table_sg * gsz) % 16 == 0 &&
                       (master == nullptr || (uintptr_t)master % 16 == 0) &&
                       (weights == nullptr || (uintptr_t)weights % 16 == 0);
  // a zero-fill workgroup clears about 64 KiB: a block of rows over all groups
  int64_t zero_rows = 0, zero_wgs = 0;
  if (zero_fill) {
    zero_rows = std::max<int64_t>(1, std::min<int64_t>(kBwdMaxIds, 65536 / std::max<int64_t>(1, groups * cols * (int64_t)gsz)));
    zero_wgs = ceil_div(row_count, zero_rows);
  }
  RTP_REQUIRE(n_ids + zero_wgs < (1ll << 31), "rtp_embedding_backward: grid too large");
  const dim3 grid((unsigned)(n_ids + zero_wgs));
  // algorithmic bytes: every upstream row read once, every named row written (or read, modified and written) once;
  // the fill of the rows nobody names is extra
  ProfileScope prof(s, "embedding_backward", (double)groups * n_ids * cols,
                    (double)groups * n_ids * cols * (esz + (zero_fill || master ? 1.0 : 2.0) * gsz) + 8.0 * n_ids);
#define RTP_EMB_BWD(T, G, V)                                                                                          \
  hipLaunchKernelGGL((embedding_bwd_kernel<T, G, V>), grid, dim3(256), 0, s, (const T*)grad_out, (long)ld_grad_out,    \
                     (int)n_ids, ids, (G*)grad_table, (long)ld_grad_table, (long)row_begin, (long)row_count, (long)cols, \
                     (long)padding_idx, scale_by_freq, zero_fill ? 1 : 0, (int)groups, (long)grad_out_sg,               \
                     (long)grad_table_sg, grad_scale, master, (T*)weights, lr, clip, store_grad, (int)zero_rows)
  if (dtype == RTP_F32) {
    if (aligned) RTP_EMB_BWD(float, float, 4); else RTP_EMB_BWD(float, float, 1);
  } else if (grad_table_f32) {
    if (aligned) RTP_EMB_BWD(bf16_t, float, 8); else RTP_EMB_BWD(bf16_t, float, 1);
  } else {
    if (aligned) RTP_EMB_BWD(bf16_t, bf16_t, 8); else RTP_EMB_BWD(bf16_t, bf16_t, 1);
  }
#undef RTP_EMB_BWD
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
