// Out-channel-sharded 2-D convolution as an implicit GEMM on the MFMA: the patch matrix
//   patches[(n*Ho + ho)*Wo + wo][(ci*kh + i)*kw + j] = x[n][ci][ho*sh - ph + i*dh][wo*sw - pw + j*dw]   (0 outside)
// is never written to memory.  One tile kernel computes  C[m][n] = sum_k A(m, k) * B(n, k)  for operands given as index
// functions; the three products of the layer are three pairs of such functions:
//   forward          y[img][co][ho][wo] = sum_k W_s[co][k] * patches[pix][k] + b_s[co]         (m = co, n = pix)
//   weight gradient  dW_s[co][k']       = sum_pix dy[img][co][ho][wo] * patches[pix][k']       (m = co, n = k')
//   input gradient   dx[img][ci][h][w]  = sum_(s,co,i,j) W_s[co][ci][i][j] * dy[img][co][ho][wo]   (m = ci, n = (img,h,w))
// A shard's weight [Co_s, Ci, kh, kw] is, as stored in its flat buffer, the row-major [Co_s, Ci*kh*kw] operand.  The
// lanes of the MFMA result run along n, which is the contiguous direction of every output (NCHW pixels, or the
// weight's k'), so stores are coalesced and the forward needs no layout copy.  Correctness first: operands are
// gathered element by element (index arithmetic per element); the reference's use of the layer is the MNIST demo.
#include <algorithm>

#include "common.h"

#include "rtp_hip.h"

namespace rtp {

typedef __attribute__((ext_vector_type(8))) __bf16 conv_bf16x8;
typedef __attribute__((ext_vector_type(16))) float conv_f32x16;

// Sizes and indices are 32-bit on the device (integer division per gathered element; the host checks the ranges);
// only the final address arithmetic is 64-bit.
struct ConvGeom {
  int n, c, h, w, kh, kw, sh, sw, ph, pw, dh, dw, ho, wo;
};

// A 4-D activation addressed by element strides (any memory format).
template <typename T>
struct Act4 {
  const T* p;
  long sn, sc, sh, sw;
  __device__ __forceinline__ T at(int n, int c, int h, int w) const { return p[n * sn + c * sc + h * sh + w * sw]; }
};

// ---- operand functions: value(group, row, k); the kernel never asks beyond rows() x depth() ----

// Rows of the weights of the shards of a run: W_g[row][k], g = group.
template <typename T>
struct WeightRows {
  const T* w;  // first shard of the run, weight at element w_off of every shard row
  long numel, kp;
  __device__ __forceinline__ T operator()(int g, int row, int k) const { return w[g * numel + (long)row * kp + k]; }
};

// patches[pix][k] (TRANSPOSED: asked as (row = k, k = pix)).
template <typename T, bool TRANSPOSED>
struct Patches {
  Act4<T> x;
  ConvGeom g;
  __device__ __forceinline__ T operator()(int, int row, int k) const {
    const int pix = TRANSPOSED ? k : row, kk = TRANSPOSED ? row : k;
    const int j = kk % g.kw, i = (kk / g.kw) % g.kh, ci = kk / (g.kw * g.kh);
    const int wo = pix % g.wo, ho = (pix / g.wo) % g.ho, n = pix / (g.wo * g.ho);
    const int h = ho * g.sh - g.ph + i * g.dh, w = wo * g.sw - g.pw + j * g.dw;
    if (h < 0 || h >= g.h || w < 0 || w >= g.w) return from_f32<T>(0.0f);
    return x.at(n, ci, h, w);
  }
};

// dy[img][co0 + g*n_s + row][ho][wo] asked as (row = co, k = pix).
template <typename T>
struct GradRowsT {
  Act4<T> dy;
  int co0, n_s, wo, howo;
  __device__ __forceinline__ T operator()(int g, int row, int k) const {
    const int img = k / howo, r = k - img * howo;
    return dy.at(img, co0 + g * n_s + row, r / wo, r % wo);
  }
};

// Input gradient, first operand: W_s[co][ci][i][j] asked as (row = ci, k = ((s*n_s + co)*kh + i)*kw + j).
template <typename T>
struct WeightByInput {
  const T* w;
  long numel;
  int n_s, c, khkw;
  __device__ __forceinline__ T operator()(int, int row, int k) const {
    const int ij = k % khkw, sco = k / khkw, s = sco / n_s, co = sco - s * n_s;
    return w[s * numel + ((long)co * c + row) * khkw + ij];
  }
};

// Input gradient, second operand: the entry of dy that patch position (i, j) of output channel co reads at input
// pixel (img, h, w), asked as (row = (img*H + h)*W + w, k as above); 0 where no output pixel reads it.
template <typename T>
struct GradByInput {
  Act4<T> dy;
  ConvGeom g;
  int co0;
  __device__ __forceinline__ T operator()(int, int row, int k) const {
    const int j = k % g.kw, i = (k / g.kw) % g.kh, sco = k / (g.kw * g.kh);
    const int w = row % g.w, h = (row / g.w) % g.h, img = row / (g.w * g.h);
    const int hn = h + g.ph - i * g.dh, wn = w + g.pw - j * g.dw;
    if (hn < 0 || wn < 0 || hn % g.sh != 0 || wn % g.sw != 0) return from_f32<T>(0.0f);
    const int ho = hn / g.sh, wo = wn / g.sw;
    if (ho >= g.ho || wo >= g.wo) return from_f32<T>(0.0f);
    return dy.at(img, co0 + sco, ho, wo);
  }
};

// ---- where a result element goes ----

// forward: y[img][co0 + g*n_s + m][ho][wo] (contiguous NCHW with `co_total` channels) = acc + bias_g[m]
template <typename T>
struct StoreNCHW {
  T* y;
  const T* bias;  // of the run's first shard (element bias_off of its row), or nullptr
  long numel;
  int co0, n_s, co_total, howo;
  __device__ __forceinline__ void operator()(int g, int, int m, int n, float v) const {
    if (bias != nullptr) v += to_f32(bias[g * numel + m]);
    const int img = n / howo, r = n - img * howo;
    y[((long)img * co_total + co0 + g * n_s + m) * howo + r] = from_f32<T>(v);
  }
  __device__ __forceinline__ void rowsum(int, int, int, float) const {}
  static constexpr bool kRowSum = false;
};

// weight gradient: grads_g[w_off + m*kp + n] (+)= acc; the row sums of the first operand are the bias gradient.
// With the contraction (the pixels) split over several workgroups, each writes its fp32 partial sums
// part[split][g][m][0 .. kp] (entry kp of a row: the partial row sum) and wgrad_reduce_kernel adds them in order.
template <typename T>
struct StoreWeightGrad {
  T* grads;  // gradient row of the run's first shard
  long numel, w_off, b_off, kp;
  int accumulate;
  float* part;  // nullptr: one workgroup per output tile, results go straight to grads
  int groups, n_s;
  __device__ __forceinline__ float* partial(int g, int split, int m) const {
    return part + (((long)split * groups + g) * n_s + m) * (kp + 1);
  }
  __device__ __forceinline__ void operator()(int g, int split, int m, int n, float v) const {
    if (part != nullptr) {
      partial(g, split, m)[n] = v;
      return;
    }
    T* dst = grads + g * numel + w_off + (long)m * kp + n;
    if (accumulate) v += to_f32(*dst);
    *dst = from_f32<T>(v);
  }
  __device__ __forceinline__ void rowsum(int g, int split, int m, float v) const {
    if (part != nullptr) {
      partial(g, split, m)[kp] = v;
      return;
    }
    if (b_off < 0) return;
    T* dst = grads + g * numel + b_off + m;
    if (accumulate) v += to_f32(*dst);
    *dst = from_f32<T>(v);
  }
  static constexpr bool kRowSum = true;
};

// grads (+)= sum over the splits, ascending, of the partial sums: one thread per entry of a shard's [n_s, kp + 1] block
template <typename T>
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(StoreWeightGrad<T> o, int splits) {
  const long per = (long)o.n_s * (o.kp + 1), total = per * o.groups;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long)gridDim.x * blockDim.x) {
    const int g = (int)(idx / per);
    const long r = idx - g * per;
    const int m = (int)(r / (o.kp + 1)), n = (int)(r - m * (o.kp + 1));
    float v = 0.0f;
    for (int sp = 0; sp < splits; ++sp) v += o.partial(g, sp, m)[n];
    T* dst;
    if (n < o.kp) {
      dst = o.grads + g * o.numel + o.w_off + (long)m * o.kp + n;
    } else {
      if (o.b_off < 0) continue;
      dst = o.grads + g * o.numel + o.b_off + m;
    }
    if (o.accumulate) v += to_f32(*dst);
    *dst = from_f32<T>(v);
  }
}

// input gradient: out[img][m][h][w] = acc + addend, out / addend in T or fp32 (the sum over rotation windows is kept
// in fp32 and rounded once)
template <typename T>
struct StoreInputGrad {
  void* out;
  const void* addend;
  int out_f32, addend_f32;
  int c, hw;
  __device__ __forceinline__ void operator()(int, int, int m, int n, float v) const {
    const int img = n / hw, r = n - img * hw;
    const long idx = ((long)img * c + m) * hw + r;
    if (addend != nullptr)
      v += addend_f32 ? reinterpret_cast<const float*>(addend)[idx] : to_f32(reinterpret_cast<const T*>(addend)[idx]);
    if (out_f32)
      reinterpret_cast<float*>(out)[idx] = v;
    else
      reinterpret_cast<T*>(out)[idx] = from_f32<T>(v);
  }
  __device__ __forceinline__ void rowsum(int, int, int, float) const {}
  static constexpr bool kRowSum = false;
};

// ---- the tile kernel: 64 x 64 outputs per workgroup, K in slabs of 32, four waves of one 32 x 32 MFMA block ----
constexpr int kConvTile = 64, kConvSlab = 32;

template <typename T>
struct ConvFrag;
template <>
struct ConvFrag<bf16_t> {
  conv_bf16x8 v;
  static constexpr int kStep = 16;  // k per MFMA step: lane group g holds k = 8g .. 8g+7
};
template <>
struct ConvFrag<float> {
  float f[4];
  static constexpr int kStep = 8;   // lane group g holds k = 4g .. 4g+3
};

__device__ __forceinline__ void conv_mma(const ConvFrag<bf16_t>& a, const ConvFrag<bf16_t>& b, conv_f32x16& c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}
__device__ __forceinline__ void conv_mma(const ConvFrag<float>& a, const ConvFrag<float>& b, conv_f32x16& c) {
#pragma unroll
  for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[e], b.f[e], c, 0, 0, 0);
}

template <typename T, class OpA, class OpB, class Out>
__global__ __launch_bounds__(256) void conv_igemm_kernel(OpA opa, OpB opb, Out out, int M, int N, int K, int splits,
                                                         int kchunk) {
  constexpr int PITCH = kConvSlab + 16 / (int)sizeof(T);  // elements; rows stay 16-byte aligned
  __shared__ __attribute__((aligned(16))) T As[kConvTile * PITCH];
  __shared__ __attribute__((aligned(16))) T Bs[kConvTile * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, li = lane & 31, g = lane >> 5;
  const int m0 = blockIdx.y * kConvTile, n0 = blockIdx.x * kConvTile;
  // blockIdx.z = (group, part of the contraction): this workgroup sums k in [kb, ke)
  const int grp = blockIdx.z / splits, split = blockIdx.z - grp * splits;
  const int kb = split * kchunk, ke = kb + kchunk < K ? kb + kchunk : K;
  const int lr = tid >> 2, lk = (tid & 3) * 8;  // the thread fills 8 consecutive k of one row of either operand
  conv_f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  float rsum = 0.0f;
  for (int k0 = kb; k0 < ke; k0 += kConvSlab) {
    T va[8], vb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = k0 + lk + e;
      va[e] = (m0 + lr < M && k < ke) ? opa(grp, m0 + lr, k) : from_f32<T>(0.0f);
      vb[e] = (n0 + lr < N && k < ke) ? opb(grp, n0 + lr, k) : from_f32<T>(0.0f);
    }
    __syncthreads();  // the previous slab has been consumed
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      As[lr * PITCH + lk + e] = va[e];
      Bs[lr * PITCH + lk + e] = vb[e];
    }
    __syncthreads();
    if (Out::kRowSum && blockIdx.x == 0 && tid < kConvTile) {
      // row sums of the first operand (a bias gradient): row tid, ascending k
      for (int k = 0; k < kConvSlab; ++k) rsum += to_f32(As[tid * PITCH + k]);
    }
    constexpr int STEP = ConvFrag<T>::kStep, VEC = 16 / (int)sizeof(T);
#pragma unroll
    for (int ks = 0; ks < kConvSlab / STEP; ++ks) {
      union {
        uint4 q;
        ConvFrag<T> f;
      } a, b;
      a.q = *reinterpret_cast<const uint4*>(&As[(wm * 32 + li) * PITCH + ks * STEP + g * VEC]);
      b.q = *reinterpret_cast<const uint4*>(&Bs[(wn * 32 + li) * PITCH + ks * STEP + g * VEC]);
      conv_mma(a.f, b.f, acc);
    }
  }
  // accumulator register r of lane (li, g): row 8*(r/4) + 4*g + r%4 of the wave's block, column li
  const int col = n0 + wn * 32 + li;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = m0 + wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
    if (row < M && col < N) out(grp, split, row, col, acc[r]);
  }
  if (Out::kRowSum && blockIdx.x == 0 && tid < kConvTile && m0 + tid < M) out.rowsum(grp, split, m0 + tid, rsum);
}

static int check_geom(const char* who, const rtp_conv_geom* geom, ConvGeom& g) {
  RTP_REQUIRE(geom, "%s: null geometry", who);
  const rtp_conv_geom& q = *geom;
  RTP_REQUIRE(q.n >= 1 && q.c >= 1 && q.h >= 1 && q.w >= 1 && q.kh >= 1 && q.kw >= 1, "%s: sizes must be >= 1", who);
  RTP_REQUIRE(q.sh >= 1 && q.sw >= 1 && q.dh >= 1 && q.dw >= 1 && q.ph >= 0 && q.pw >= 0,
              "%s: stride and dilation must be >= 1, padding >= 0", who);
  const int64_t lim = (int64_t)1 << 30;  // every index of the three products stays within 32 bits
  RTP_REQUIRE(q.sh < lim && q.sw < lim && q.dh < lim && q.dw < lim && q.ph < lim && q.pw < lim && q.ho >= 1 &&
                  q.wo >= 1 && q.n * q.h * q.w < lim && q.n * q.ho * q.wo < lim && q.c * q.kh * q.kw < lim &&
                  q.dh * q.kh < lim && q.dw * q.kw < lim && q.ho * q.sh < lim && q.wo * q.sw < lim,
              "%s: geometry beyond the 32-bit index range of the kernels", who);
  g = ConvGeom{(int)q.n, (int)q.c, (int)q.h, (int)q.w, (int)q.kh, (int)q.kw, (int)q.sh, (int)q.sw,
               (int)q.ph, (int)q.pw, (int)q.dh, (int)q.dw, (int)q.ho, (int)q.wo};
  const long span_h = (long)g.h + 2 * g.ph - (long)g.dh * (g.kh - 1) - 1, span_w = (long)g.w + 2 * g.pw - (long)g.dw * (g.kw - 1) - 1;
  RTP_REQUIRE(span_h >= 0 && span_w >= 0, "%s: kernel larger than the padded input", who);
  RTP_REQUIRE(g.ho == span_h / g.sh + 1 && g.wo == span_w / g.sw + 1,
              "%s: output size %lld x %lld does not match the geometry (expected %lld x %lld)", who, (long long)g.ho,
              (long long)g.wo, (long long)(span_h / g.sh + 1), (long long)(span_w / g.sw + 1));
  return RTP_OK;
}

static int check_run(const char* who, int dtype, int64_t numel, int64_t shards, int64_t w_off, int64_t bias_off,
                     int64_t n_s, const ConvGeom& g) {
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "%s: unknown dtype %d", who, dtype);
  const long kp = (long)g.c * g.kh * g.kw;
  RTP_REQUIRE(shards >= 1 && shards < 65536 && n_s >= 1 && shards * n_s * g.kh * g.kw < ((int64_t)1 << 30),
              "%s: shards %lld, channels per shard %lld", who, (long long)shards, (long long)n_s);
  RTP_REQUIRE(w_off >= 0 && w_off + n_s * kp <= numel, "%s: the weight [%lld, %lld] at %lld does not fit a shard row of %lld",
              who, (long long)n_s, (long long)kp, (long long)w_off, (long long)numel);
  RTP_REQUIRE(bias_off < 0 || bias_off + n_s <= numel, "%s: the bias at %lld does not fit a shard row of %lld", who,
              (long long)bias_off, (long long)numel);
  return RTP_OK;
}

template <typename T, class OpA, class OpB, class Out>
static int launch_igemm(hipStream_t st, const char* name, OpA a, OpB b, Out o, long M, long N, long K, long groups,
                        double bytes, long splits = 1, long kchunk = 0) {
  const long tm = ceil_div(M, kConvTile), tn = ceil_div(N, kConvTile);
  RTP_REQUIRE(tn < (1l << 31) && tm < 65536 && groups * splits < 65536, "%s: grid %ld x %ld x %ld too large", name, tn,
              tm, groups * splits);
  if (splits == 1) kchunk = ceil_div(K, kConvSlab) * kConvSlab;
  ProfileScope prof(st, name, 2.0 * (double)M * (double)N * (double)K * (double)groups, bytes);
  RTP_REQUIRE(M < (1l << 30) && N < (1l << 30) && K < (1l << 30), "%s: product %ld x %ld x %ld beyond 32-bit indices", name,
              M, N, K);
  hipLaunchKernelGGL((conv_igemm_kernel<T, OpA, OpB, Out>), dim3((unsigned)tn, (unsigned)tm, (unsigned)(groups * splits)),
                     dim3(256), 0, st, a, b, o, (int)M, (int)N, (int)K, (int)splits, (int)kchunk);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

template <typename T>
static int conv_fwd(hipStream_t st, const void* x, const int64_t* sx, const ConvGeom& g, const void* w, int64_t numel,
                    int64_t shards, int64_t w_off, int64_t bias_off, int64_t n_s, void* y, int64_t co_first,
                    int64_t co_total) {
  const long kp = (long)g.c * g.kh * g.kw, pix = (long)g.n * g.ho * g.wo;
  const T* wt = reinterpret_cast<const T*>(w);
  WeightRows<T> a{wt + w_off, numel, kp};
  Patches<T, false> b{Act4<T>{reinterpret_cast<const T*>(x), sx[0], sx[1], sx[2], sx[3]}, g};
  StoreNCHW<T> o{reinterpret_cast<T*>(y), bias_off >= 0 ? wt + bias_off : nullptr, numel, (int)co_first, (int)n_s,
                 (int)co_total, g.ho * g.wo};
  const double bytes = sizeof(T) * ((double)g.n * g.c * g.h * g.w + (double)shards * n_s * (kp + pix));
  return launch_igemm<T>(st, "conv2d_fwd", a, b, o, n_s, pix, kp, shards, bytes);
}

// The weight gradient contracts over all pixels of the batch and has few outputs: the contraction is dealt over
// `splits` workgroups per output tile (about four workgroups per CU in all, at least 8 slabs each).
struct WgradSplit {
  long splits, kchunk;
  size_t workspace;
};
static WgradSplit wgrad_split(const ConvGeom& g, int64_t shards, int64_t n_s) {
  const long kp = (long)g.c * g.kh * g.kw, pix = (long)g.n * g.ho * g.wo;
  const long tiles = ceil_div(n_s, kConvTile) * ceil_div(kp, kConvTile) * shards, slabs = ceil_div(pix, kConvSlab);
  long want = std::min<long>(ceil_div(1024, tiles), std::max<long>(1, slabs / 8));
  want = std::max<long>(1, std::min<long>(want, 65535 / shards));
  WgradSplit r;
  r.kchunk = ceil_div(slabs, want) * kConvSlab;
  r.splits = ceil_div(pix, r.kchunk);
  r.workspace = r.splits > 1 ? (size_t)r.splits * shards * n_s * (kp + 1) * sizeof(float) : 0;
  return r;
}

template <typename T>
static int conv_wgrad(hipStream_t st, const void* dy, const int64_t* sdy, const void* x, const int64_t* sx,
                      const ConvGeom& g, void* grads, int64_t numel, int64_t shards, int64_t w_off, int64_t bias_off,
                      int64_t n_s, int64_t co_first, int accumulate, void* workspace, size_t workspace_bytes) {
  const long kp = (long)g.c * g.kh * g.kw, pix = (long)g.n * g.ho * g.wo;
  const WgradSplit sp = wgrad_split(g, shards, n_s);
  if (workspace_bytes < sp.workspace || (sp.workspace && workspace == nullptr))
    return fail(RTP_ERR_WORKSPACE, "rtp_conv2d_wgrad: workspace %zu < required %zu", workspace_bytes, sp.workspace);
  GradRowsT<T> a{Act4<T>{reinterpret_cast<const T*>(dy), sdy[0], sdy[1], sdy[2], sdy[3]}, (int)co_first, (int)n_s,
                 g.wo, g.ho * g.wo};
  Patches<T, true> b{Act4<T>{reinterpret_cast<const T*>(x), sx[0], sx[1], sx[2], sx[3]}, g};
  StoreWeightGrad<T> o{reinterpret_cast<T*>(grads), numel, w_off, bias_off, kp, accumulate,
                       sp.splits > 1 ? reinterpret_cast<float*>(workspace) : nullptr, (int)shards, (int)n_s};
  const double bytes = sizeof(T) * ((double)g.n * g.c * g.h * g.w + (double)shards * n_s * (kp + pix));
  if (int rc = launch_igemm<T>(st, "conv2d_wgrad", a, b, o, n_s, kp, pix, shards, bytes, sp.splits, sp.kchunk)) return rc;
  if (sp.splits > 1) {
    const long total = (long)shards * n_s * (kp + 1);
    ProfileScope prof(st, "conv2d_wgrad_reduce", 0.0, (double)sp.workspace + (double)total * sizeof(T));
    hipLaunchKernelGGL(wgrad_reduce_kernel<T>, dim3((unsigned)std::min<long>(4096, ceil_div(total, 256))), dim3(256), 0, st,
                       o, (int)sp.splits);
    RTP_LAUNCH_CHECK();
  }
  return RTP_OK;
}

template <typename T>
static int conv_dgrad(hipStream_t st, const void* dy, const int64_t* sdy, const ConvGeom& g, const void* w,
                      int64_t numel, int64_t shards, int64_t w_off, int64_t n_s, int64_t co_first, void* dx, int dx_f32,
                      const void* addend, int addend_f32) {
  const int khkw = g.kh * g.kw;
  const long inpix = (long)g.n * g.h * g.w;
  WeightByInput<T> a{reinterpret_cast<const T*>(w) + w_off, numel, (int)n_s, g.c, khkw};
  GradByInput<T> b{Act4<T>{reinterpret_cast<const T*>(dy), sdy[0], sdy[1], sdy[2], sdy[3]}, g, (int)co_first};
  StoreInputGrad<T> o{dx, addend, dx_f32, addend_f32, g.c, g.h * g.w};
  const double bytes = sizeof(T) * ((double)g.n * g.c * g.h * g.w +
                                    (double)shards * n_s * ((double)g.c * khkw + (double)g.n * g.ho * g.wo));
  return launch_igemm<T>(st, "conv2d_dgrad", a, b, o, g.c, inpix, shards * n_s * khkw, 1, bytes);
}

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_conv2d_fwd(void* stream, int dtype, const void* x, int64_t sx_n, int64_t sx_c, int64_t sx_h,
                              int64_t sx_w, const rtp_conv_geom* geom, const void* w, int64_t numel, int64_t shards,
                              int64_t w_off, int64_t bias_off, int64_t n_s, void* y, int64_t co_first,
                              int64_t co_total) {
  ConvGeom g;
  if (int rc = check_geom("rtp_conv2d_fwd", geom, g)) return rc;
  if (int rc = check_run("rtp_conv2d_fwd", dtype, numel, shards, w_off, bias_off, n_s, g)) return rc;
  RTP_REQUIRE(x && w && y, "rtp_conv2d_fwd: null pointer");
  RTP_REQUIRE(co_first >= 0 && co_first + shards * n_s <= co_total, "rtp_conv2d_fwd: channels %lld .. %lld of %lld",
              (long long)co_first, (long long)(co_first + shards * n_s), (long long)co_total);
  const int64_t sx[4] = {sx_n, sx_c, sx_h, sx_w};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == RTP_F32)
    return conv_fwd<float>(st, x, sx, g, w, numel, shards, w_off, bias_off, n_s, y, co_first, co_total);
  return conv_fwd<bf16_t>(st, x, sx, g, w, numel, shards, w_off, bias_off, n_s, y, co_first, co_total);
}

extern "C" int rtp_conv2d_wgrad(void* stream, int dtype, const void* dy, int64_t sdy_n, int64_t sdy_c, int64_t sdy_h,
                                int64_t sdy_w, const void* x, int64_t sx_n, int64_t sx_c, int64_t sx_h, int64_t sx_w,
                                const rtp_conv_geom* geom, void* grads, int64_t numel, int64_t shards, int64_t w_off,
                                int64_t bias_off, int64_t n_s, int64_t co_first, int accumulate, void* workspace,
                                size_t workspace_bytes) {
  ConvGeom g;
  if (int rc = check_geom("rtp_conv2d_wgrad", geom, g)) return rc;
  if (int rc = check_run("rtp_conv2d_wgrad", dtype, numel, shards, w_off, bias_off, n_s, g)) return rc;
  RTP_REQUIRE(dy && x && grads && co_first >= 0, "rtp_conv2d_wgrad: null pointer or negative channel offset");
  const int64_t sdy[4] = {sdy_n, sdy_c, sdy_h, sdy_w}, sx[4] = {sx_n, sx_c, sx_h, sx_w};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == RTP_F32)
    return conv_wgrad<float>(st, dy, sdy, x, sx, g, grads, numel, shards, w_off, bias_off, n_s, co_first, accumulate,
                             workspace, workspace_bytes);
  return conv_wgrad<bf16_t>(st, dy, sdy, x, sx, g, grads, numel, shards, w_off, bias_off, n_s, co_first, accumulate,
                            workspace, workspace_bytes);
}

extern "C" size_t rtp_conv2d_wgrad_workspace_bytes(const rtp_conv_geom* geom, int64_t shards, int64_t n_s) {
  ConvGeom g;
  if (check_geom("rtp_conv2d_wgrad_workspace_bytes", geom, g) != RTP_OK || shards < 1 || shards >= 65536 || n_s < 1)
    return 0;
  return wgrad_split(g, shards, n_s).workspace;
}

extern "C" int rtp_conv2d_dgrad(void* stream, int dtype, const void* dy, int64_t sdy_n, int64_t sdy_c, int64_t sdy_h,
                                int64_t sdy_w, const rtp_conv_geom* geom, const void* w, int64_t numel, int64_t shards,
                                int64_t w_off, int64_t n_s, int64_t co_first, void* dx, int dx_f32, const void* addend,
                                int addend_f32) {
  ConvGeom g;
  if (int rc = check_geom("rtp_conv2d_dgrad", geom, g)) return rc;
  if (int rc = check_run("rtp_conv2d_dgrad", dtype, numel, shards, w_off, -1, n_s, g)) return rc;
  RTP_REQUIRE(dy && w && dx && co_first >= 0, "rtp_conv2d_dgrad: null pointer or negative channel offset");
  const int64_t sdy[4] = {sdy_n, sdy_c, sdy_h, sdy_w};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == RTP_F32)
    return conv_dgrad<float>(st, dy, sdy, g, w, numel, shards, w_off, n_s, co_first, dx, 1, addend, 1);
  return conv_dgrad<bf16_t>(st, dy, sdy, g, w, numel, shards, w_off, n_s, co_first, dx, dx_f32, addend, addend_f32);
}
