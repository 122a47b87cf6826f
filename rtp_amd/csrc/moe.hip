// GShard top-2 routing as compact per-token records (expert, slot, weight) instead of dense
// [S,E,C] one-hot tensors, and the dispatch / combine row moves that use them.
#include "common.h"

#include <cfloat>

namespace rtp {

constexpr int kMaxExperts = 64;
constexpr int kTok = 256;  // tokens per workgroup

// Phase 1: per token softmax, first choice (argmax of the probabilities), second choice (argmax of
// logits+noise with the first choice excluded); per workgroup, the stable rank of each token among
// the tokens of the same workgroup that picked the same expert, and the per-expert totals.
__global__ __launch_bounds__(kTok) void route_choose_kernel(const float* logits, const float* noise, long S, int E,
                                                            int* expert, int* rank, float* gates, int* slot_token,
                                                            int* blockcnt, float* blockgate) {
  __shared__ int wcnt[2][4][kMaxExperts];
  __shared__ float wgate[4][kMaxExperts];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const long s = (long)blockIdx.x * kTok + tid;
  const bool valid = s < S;
  int e1 = -1, e2 = -1;
  float mx = -INFINITY, sum = 0.0f;
  if (valid) {
    const float* lg = logits + s * E;
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, lg[e]);
    for (int e = 0; e < E; ++e) sum += expf(lg[e] - mx);
    float best = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float gv = expf(lg[e] - mx) / sum;
      gates[s * E + e] = gv;
      if (e1 < 0 || gv > best) {
        best = gv;
        e1 = e;
      }
    }
    const float* nz = noise + s * E;
    float best2 = -INFINITY;
    e2 = 0;
    bool have = false;
    for (int e = 0; e < E; ++e) {
      if (e == e1) continue;
      const float v = lg[e] + nz[e];
      if (!have || v > best2) {
        best2 = v;
        e2 = e;
        have = true;
      }
    }
    // C = 2S/E slots per expert, so the E*C <= 2S entries of slot_token are cleared two per token.
    slot_token[2 * s] = -1;
    slot_token[2 * s + 1] = -1;
  }
  const unsigned long long lt = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int r1 = 0, r2 = 0;
  for (int e = 0; e < E; ++e) {
    const unsigned long long b1 = __ballot(valid && e1 == e);
    const unsigned long long b2 = __ballot(valid && e2 == e);
    if (e1 == e) r1 = __popcll(b1 & lt);
    if (e2 == e) r2 = __popcll(b2 & lt);
    if (lane == 0) {
      wcnt[0][w][e] = __popcll(b1);
      wcnt[1][w][e] = __popcll(b2);
    }
    const float gsum = wave_sum(valid ? gates[s * E + e] : 0.0f);
    if (lane == 0) wgate[w][e] = gsum;
  }
  __syncthreads();
  if (valid) {
    for (int ww = 0; ww < w; ++ww) {
      r1 += wcnt[0][ww][e1];
      r2 += wcnt[1][ww][e2];
    }
    expert[2 * s] = e1;
    expert[2 * s + 1] = e2;
    rank[2 * s] = r1;
    rank[2 * s + 1] = r2;
  }
  if (tid < E) {
    const long o = (long)blockIdx.x * E + tid;
    blockcnt[2 * o] = wcnt[0][0][tid] + wcnt[0][1][tid] + wcnt[0][2][tid] + wcnt[0][3][tid];
    blockcnt[2 * o + 1] = wcnt[1][0][tid] + wcnt[1][1][tid] + wcnt[1][2][tid] + wcnt[1][3][tid];
    blockgate[o] = (wgate[0][tid] + wgate[1][tid]) + (wgate[2][tid] + wgate[3][tid]);
  }
}

// Phase 2 (one workgroup): exclusive scan of the per-workgroup totals per expert, the grand totals and
// the auxiliary loss  l_aux = mean_e( mean_s gates[s,e] * mean_s [e1(s)==e] ).
__global__ __launch_bounds__(kMaxExperts) void route_scan_kernel(int* blockcnt, const float* blockgate, long nblocks,
                                                                 long S, int E, int* counts, float* l_aux,
                                                                 bf16_t* l_aux_bf16) {
  __shared__ float term[kMaxExperts];
  const int e = threadIdx.x;
  if (e < E) {
    int run1 = 0, run2 = 0;
    float gs = 0.0f;
    for (long b = 0; b < nblocks; ++b) {
      const long o = b * E + e;
      const int c1 = blockcnt[2 * o], c2 = blockcnt[2 * o + 1];
      blockcnt[2 * o] = run1;
      blockcnt[2 * o + 1] = run2;
      run1 += c1;
      run2 += c2;
      gs += blockgate[o];
    }
    counts[e] = run1;
    counts[E + e] = run2;
    term[e] = (gs / (float)S) * ((float)run1 / (float)S);
  }
  __syncthreads();
  if (e == 0) {
    float t = 0.0f;
    for (int i = 0; i < E; ++i) t += term[i];
    *l_aux = t / (float)E;
    if (l_aux_bf16 != nullptr) *l_aux_bf16 = from_f32<bf16_t>(t / (float)E);
  }
}

// Phase 3: global location = scanned base + in-workgroup rank (+ all first choices of that expert, for a
// second choice); capacity drop; renormalised weights; slot -> token map.
__global__ __launch_bounds__(kTok) void route_finalize_kernel(const float* gates, const int* expert, const int* rank,
                                                              const int* blockbase, const int* counts, long S, int E,
                                                              int C, int* slot, int* keep, float* weight,
                                                              int* slot_token) {
  const long s = (long)blockIdx.x * kTok + threadIdx.x;
  if (s >= S) return;
  const int e1 = expert[2 * s], e2 = expert[2 * s + 1];
  const long o1 = (long)blockIdx.x * E + e1, o2 = (long)blockIdx.x * E + e2;
  const int loc1 = blockbase[2 * o1] + rank[2 * s];
  const int loc2 = blockbase[2 * o2 + 1] + rank[2 * s + 1] + counts[e2];
  bool k1 = loc1 < C, k2 = loc2 < C;
  const float g1 = k1 ? gates[s * E + e1] : 0.0f;
  const float g2 = k2 ? gates[s * E + e2] : 0.0f;
  const float den = fmaxf(g1 + g2, FLT_EPSILON);
  const float w1 = g1 / den, w2 = g2 / den;
  // The reference dispatches where the combine weight is non-zero.
  k1 = k1 && w1 != 0.0f;
  k2 = k2 && w2 != 0.0f;
  slot[2 * s] = k1 ? loc1 : 0;
  slot[2 * s + 1] = k2 ? loc2 : 0;
  keep[2 * s] = k1;
  keep[2 * s + 1] = k2;
  weight[2 * s] = k1 ? w1 : 0.0f;
  weight[2 * s + 1] = k2 ? w2 : 0.0f;
  if (k1) slot_token[(long)e1 * C + loc1] = (int)s;
  if (k2) slot_token[(long)e2 * C + loc2] = (int)s;
}

__global__ __launch_bounds__(kTok) void route_bwd_kernel(const float* gates, const int* expert, const int* keep,
                                                         const int* counts, const float* d_weight,
                                                         const float* d_l_aux, long S, int E, float* d_logits) {
  const long s = (long)blockIdx.x * kTok + threadIdx.x;
  if (s >= S) return;
  const int e1 = expert[2 * s], e2 = expert[2 * s + 1];
  const bool k1 = keep[2 * s], k2 = keep[2 * s + 1];
  const float* g = gates + s * E;
  const float g1 = k1 ? g[e1] : 0.0f, g2 = k2 ? g[e2] : 0.0f;
  const float raw = g1 + g2;
  const float den = fmaxf(raw, FLT_EPSILON);
  const float dw1 = d_weight[2 * s], dw2 = d_weight[2 * s + 1];
  const float dden = raw >= FLT_EPSILON ? -(dw1 * g1 + dw2 * g2) / (den * den) : 0.0f;
  const float dg1 = k1 ? dw1 / den + dden : 0.0f;
  const float dg2 = k2 ? dw2 / den + dden : 0.0f;
  const float dl = d_l_aux ? *d_l_aux : 0.0f;
  const float aux_scale = dl / ((float)E * (float)S * (float)S);
  float dot = 0.0f;
  for (int e = 0; e < E; ++e) {
    float dge = aux_scale * (float)counts[e];
    if (e == e1) dge += dg1;
    if (e == e2) dge += dg2;
    dot += dge * g[e];
  }
  for (int e = 0; e < E; ++e) {
    float dge = aux_scale * (float)counts[e];
    if (e == e1) dge += dg1;
    if (e == e2) dge += dg2;
    d_logits[s * E + e] = g[e] * (dge - dot);
  }
}

// out[row,:] = x[token(row),:] (* weight of the choice that put the token there), zero if the slot is
// empty.  One workgroup per (slot row, column chunk).
template <typename T>
__global__ __launch_bounds__(256) void dispatch_kernel(const T* x, long ld_x, const int* slot_token,
                                                       const int* expert, const int* slot, const float* weight,
                                                       long capacity, long cols, T* out, long ld_out) {
  const long row = blockIdx.x;
  const int tok = slot_token[row];
  T* dst = out + row * ld_out;
  if (tok < 0) {
    for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < cols; c += (long)gridDim.y * 256) dst[c] = (T)0.0f;
    return;
  }
  const T* src = x + (long)tok * ld_x;
  if (weight) {
    const int e = (int)(row / capacity), c0 = (int)(row % capacity);
    const int j = (expert[2 * tok] == e && slot[2 * tok] == c0 && weight[2 * tok] != 0.0f) ? 0 : 1;
    const float w = weight[2 * tok + j];
    for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < cols; c += (long)gridDim.y * 256)
      dst[c] = from_f32<T>(w * to_f32(src[c]));
  } else {
    for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < cols; c += (long)gridDim.y * 256) dst[c] = src[c];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void combine_kernel(const T* y, long ld_y, const int* expert, const int* slot,
                                                      const int* keep, const float* weight, long capacity, long cols,
                                                      T* out, long ld_out) {
  const long s = blockIdx.x;
  const bool k1 = keep[2 * s], k2 = keep[2 * s + 1];
  const T* y1 = y + ((long)expert[2 * s] * capacity + slot[2 * s]) * ld_y;
  const T* y2 = y + ((long)expert[2 * s + 1] * capacity + slot[2 * s + 1]) * ld_y;
  const float w1 = weight ? weight[2 * s] : 1.0f, w2 = weight ? weight[2 * s + 1] : 1.0f;
  T* dst = out + s * ld_out;
  for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < cols; c += (long)gridDim.y * 256) {
    float v = 0.0f;
    if (k1) v += w1 * to_f32(y1[c]);
    if (k2) v += w2 * to_f32(y2[c]);
    dst[c] = from_f32<T>(v);
  }
}

// One wavefront per (token, choice): dw = <dout[token,:], y[slot row,:]>.
template <typename T>
__global__ __launch_bounds__(256) void combine_dweight_kernel(const T* dout, long ld_dout, const T* y, long ld_y,
                                                              const int* expert, const int* slot, const int* keep,
                                                              long S, long capacity, long cols, float* dweight) {
  const int lane = threadIdx.x & 63;
  const long idx = (long)blockIdx.x * 4 + (threadIdx.x >> 6);  // = 2*s + j
  if (idx >= 2 * S) return;
  float acc = 0.0f;
  if (keep[idx]) {
    const T* a = dout + (idx >> 1) * ld_dout;
    const T* b = y + ((long)expert[idx] * capacity + slot[idx]) * ld_y;
    for (long c = lane; c < cols; c += kWave) acc += to_f32(a[c]) * to_f32(b[c]);
  }
  acc = wave_sum(acc);
  if (lane == 0) dweight[idx] = acc;
}

struct RouteLayout {
  size_t rank, blockcnt, blockgate, total;
  long nblocks;
};
static RouteLayout route_layout(int64_t s, int64_t e) {
  RouteLayout L;
  L.nblocks = (long)ceil_div(s, kTok);
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  L.rank = 0;
  L.blockcnt = up((size_t)s * 2 * 4);
  L.blockgate = L.blockcnt + up((size_t)L.nblocks * e * 2 * 4);
  L.total = L.blockgate + up((size_t)L.nblocks * e * 4);
  return L;
}

static unsigned col_chunks(int64_t cols) { return (unsigned)std::min<int64_t>(8, std::max<int64_t>(1, cols / 1024)); }

}  // namespace rtp

using namespace rtp;

extern "C" size_t rtp_top2_route_workspace_bytes(int64_t s, int64_t e) {
  if (s <= 0 || e <= 0) return 256;
  return route_layout(s, e).total;
}

extern "C" int rtp_top2_route(void* stream, const float* logits, const float* noise, int64_t s, int64_t e,
                              int32_t* expert, int32_t* slot, int32_t* keep, float* weight, float* gates,
                              int32_t* slot_token, float* l_aux, int32_t* counts, void* workspace,
                              size_t workspace_bytes, void* l_aux_bf16) {
  RTP_REQUIRE(logits && noise && expert && slot && keep && weight && gates && slot_token && l_aux && counts &&
                  workspace,
              "rtp_top2_route: null pointer");
  RTP_REQUIRE(s >= 1 && e >= 2 && e <= kMaxExperts, "rtp_top2_route: need S >= 1 and 2 <= E <= %d (S=%lld E=%lld)",
              kMaxExperts, (long long)s, (long long)e);
  RTP_REQUIRE(s % e == 0, "rtp_top2_route: S=%lld is not a multiple of E=%lld", (long long)s, (long long)e);
  RTP_REQUIRE(s < (1ll << 30), "rtp_top2_route: S too large");
  RTP_REQUIRE((uintptr_t)workspace % 256 == 0, "rtp_top2_route: workspace must be 256-byte aligned");
  const RouteLayout L = route_layout(s, e);
  if (workspace_bytes < L.total)
    return fail(RTP_ERR_WORKSPACE, "rtp_top2_route: workspace %zu < required %zu", workspace_bytes, L.total);
  char* w = (char*)workspace;
  int* rank = (int*)(w + L.rank);
  int* blockcnt = (int*)(w + L.blockcnt);
  float* blockgate = (float*)(w + L.blockgate);
  const int C = (int)(2 * s / e);
  hipStream_t st = (hipStream_t)stream;
  // three launches booked as one routing pass: reads logits+noise, writes gates and the compact records
  ProfileScope prof(st, "top2_route", 0.0, (double)s * e * 12.0 + (double)s * 40.0);
  hipLaunchKernelGGL(route_choose_kernel, dim3((unsigned)L.nblocks), dim3(kTok), 0, st, logits, noise, (long)s,
                     (int)e, expert, rank, gates, slot_token, blockcnt, blockgate);
  RTP_LAUNCH_CHECK();
  hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(kMaxExperts), 0, st, blockcnt, blockgate, L.nblocks, (long)s,
                     (int)e, counts, l_aux, (bf16_t*)l_aux_bf16);
  RTP_LAUNCH_CHECK();
  hipLaunchKernelGGL(route_finalize_kernel, dim3((unsigned)L.nblocks), dim3(kTok), 0, st, gates, expert, rank,
                     blockcnt, counts, (long)s, (int)e, C, slot, keep, weight, slot_token);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_top2_route_bwd(void* stream, const float* gates, const int32_t* expert, const int32_t* keep,
                                  const int32_t* counts, const float* d_weight, const float* d_l_aux, int64_t s,
                                  int64_t e, float* d_logits) {
  RTP_REQUIRE(gates && expert && keep && counts && d_weight && d_logits, "rtp_top2_route_bwd: null pointer");
  RTP_REQUIRE(s >= 1 && e >= 2 && e <= kMaxExperts, "rtp_top2_route_bwd: bad shape S=%lld E=%lld", (long long)s,
              (long long)e);
  hipLaunchKernelGGL(route_bwd_kernel, dim3((unsigned)ceil_div(s, kTok)), dim3(kTok), 0, (hipStream_t)stream, gates,
                     expert, keep, counts, d_weight, d_l_aux, (long)s, (int)e, d_logits);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_moe_dispatch(void* stream, int dtype, const void* x, int64_t ld_x, const int32_t* slot_token,
                                const int32_t* expert, const int32_t* slot, const float* weight, int64_t n_slots,
                                int64_t capacity, int64_t cols, void* out, int64_t ld_out) {
  RTP_REQUIRE(x && slot_token && out, "rtp_moe_dispatch: null pointer");
  RTP_REQUIRE(!weight || (expert && slot), "rtp_moe_dispatch: weight needs expert and slot");
  RTP_REQUIRE(n_slots >= 0 && n_slots < (1ll << 31) && capacity >= 1 && cols >= 0 && ld_x >= cols && ld_out >= cols,
              "rtp_moe_dispatch: bad shape");
  if (n_slots == 0 || cols == 0) return RTP_OK;
  dim3 grid((unsigned)n_slots, col_chunks(cols));
  ProfileScope prof((hipStream_t)stream, "moe_dispatch", 0.0, 2.0 * (double)n_slots * cols * (dtype == RTP_F32 ? 4 : 2));
#define A_(T) (const T*)x, (long)ld_x, slot_token, expert, slot, weight, (long)capacity, (long)cols, (T*)out, (long)ld_out
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(dispatch_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, A_(float));
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(dispatch_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, A_(bf16_t));
  else
    return fail(RTP_ERR_ARG, "rtp_moe_dispatch: unknown dtype %d", dtype);
#undef A_
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_moe_combine(void* stream, int dtype, const void* y, int64_t ld_y, const int32_t* expert,
                               const int32_t* slot, const int32_t* keep, const float* weight, int64_t s,
                               int64_t capacity, int64_t cols, void* out, int64_t ld_out) {
  RTP_REQUIRE(y && expert && slot && keep && out, "rtp_moe_combine: null pointer");
  RTP_REQUIRE(s >= 0 && s < (1ll << 31) && capacity >= 1 && cols >= 0 && ld_y >= cols && ld_out >= cols,
              "rtp_moe_combine: bad shape");
  if (s == 0 || cols == 0) return RTP_OK;
  dim3 grid((unsigned)s, col_chunks(cols));
  ProfileScope prof((hipStream_t)stream, "moe_combine", 4.0 * (double)s * cols, 3.0 * (double)s * cols * (dtype == RTP_F32 ? 4 : 2));
#define A_(T) (const T*)y, (long)ld_y, expert, slot, keep, weight, (long)capacity, (long)cols, (T*)out, (long)ld_out
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(combine_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, A_(float));
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(combine_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, A_(bf16_t));
  else
    return fail(RTP_ERR_ARG, "rtp_moe_combine: unknown dtype %d", dtype);
#undef A_
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_moe_combine_dweight(void* stream, int dtype, const void* dout, int64_t ld_dout, const void* y,
                                       int64_t ld_y, const int32_t* expert, const int32_t* slot, const int32_t* keep,
                                       int64_t s, int64_t capacity, int64_t cols, float* dweight) {
  RTP_REQUIRE(dout && y && expert && slot && keep && dweight, "rtp_moe_combine_dweight: null pointer");
  RTP_REQUIRE(s >= 0 && s < (1ll << 30) && capacity >= 1 && cols >= 0 && ld_dout >= cols && ld_y >= cols,
              "rtp_moe_combine_dweight: bad shape");
  if (s == 0) return RTP_OK;
  dim3 grid((unsigned)ceil_div(2 * s, 4));
#define A_(T) (const T*)dout, (long)ld_dout, (const T*)y, (long)ld_y, expert, slot, keep, (long)s, (long)capacity, (long)cols, dweight
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(combine_dweight_kernel<float>, grid, dim3(256), 0, (hipStream_t)stream, A_(float));
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(combine_dweight_kernel<bf16_t>, grid, dim3(256), 0, (hipStream_t)stream, A_(bf16_t));
  else
    return fail(RTP_ERR_ARG, "rtp_moe_combine_dweight: unknown dtype %d", dtype);
#undef A_
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
