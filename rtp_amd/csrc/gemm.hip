// LDS-staged MFMA GEMM for gfx950 (fp32 via v_mfma_f32_32x32x2_f32, bf16 via v_mfma_f32_32x32x16_bf16)
// with the four operand layouts the rotated layers need (forward X W^T, input gradient dY W, weight
// gradient dY^T X, batched q k^T / p v) and a fused epilogue (accumulate, bias, ReLU, ReLU-mask).
//
// Work decomposition: 256 threads = 4 wavefronts in a 2x2 arrangement over a BM x BN output tile;
// each wavefront owns (BM/2)x(BN/2) as 32x32 MFMA blocks with fp32 accumulators in VGPRs.  The K loop
// moves 64-byte-per-row slabs (32 bf16 / 16 fp32 values of k) global -> registers -> LDS, double
// buffered in LDS so one barrier per slab suffices; the global loads of slab t+1 are in flight while
// the MFMAs of slab t run.
#include "common.h"

namespace rtp {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct GemmArgs {
  const char* a;
  const char* b;
  char* c_out;
  const char* c_in;
  const char* bias;
  const char* gate;
  int m, n, k;
  long lda, ldb, ldc, ld_cin, ld_gate;
  int zdiv;
  long a_so, a_si, b_so, b_si, c_so, c_si, cin_so, cin_si, gate_so, gate_si, bias_so, bias_si;
  float alpha;
  int flags;
  int vec_a, vec_b;
  int tiles_m, tiles_n;
};

constexpr int kThreads = 256;
constexpr int kRowPitchKC = 80;  // bytes per tile row when k is contiguous: 64 data + 16 pad

// Moves one R x BK operand slab global -> registers -> LDS.
//   KC  (k contiguous in memory): LDS holds [row][k], row pitch 80 bytes.
//   !KC (rows contiguous in memory): LDS holds [k][row], k pitch R*sizeof(T)+16 bytes.
template <typename T, int R, bool KC>
struct SlabLoader {
  static constexpr int VEC = 16 / sizeof(T);
  static constexpr int BK = 4 * VEC;
  static constexpr int NV = R * 4 / kThreads;
  static constexpr int RV = R / VEC;  // vectors per k line when rows are contiguous
  static constexpr int PITCH = KC ? kRowPitchKC : (R * (int)sizeof(T) + 16);
  static constexpr int BYTES = KC ? R * kRowPitchKC : BK * PITCH;
  uint4 reg[NV];

  __device__ __forceinline__ void load(const T* base, long ld, int row0, int rows, int k0, int kdim,
                                       bool vec_ok, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * kThreads;
      union {
        uint4 q;
        T e[VEC];
      } u;
      if (KC) {
        const int row = row0 + (v >> 2);
        const int k = k0 + (v & 3) * VEC;
        const T* src = base + (long)row * ld + k;
        if (vec_ok && row < rows && k + VEC <= kdim) {
          u.q = *reinterpret_cast<const uint4*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) u.e[e] = (row < rows && k + e < kdim) ? src[e] : (T)0.0f;
        }
      } else {
        const int k = k0 + v / RV;
        const int row = row0 + (v % RV) * VEC;
        const T* src = base + (long)k * ld + row;
        if (vec_ok && k < kdim && row + VEC <= rows) {
          u.q = *reinterpret_cast<const uint4*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) u.e[e] = (k < kdim && row + e < rows) ? src[e] : (T)0.0f;
        }
      }
      reg[i] = u.q;
    }
  }

  __device__ __forceinline__ void store(char* lds, int tid) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * kThreads;
      char* dst = KC ? lds + (v >> 2) * kRowPitchKC + (v & 3) * 16 : lds + (v / RV) * PITCH + (v % RV) * 16;
      *reinterpret_cast<uint4*>(dst) = reg[i];
    }
  }
};

// The per-lane MFMA operand: VEC consecutive k values of one tile row.
template <typename T>
struct Frag;
template <>
struct Frag<bf16_t> {
  bf16x8 v;
};
template <>
struct Frag<float> {
  float f[4];
};

// Lane (li = lane%32, g = lane/32) reads row `row` of the slab, k = (2*ks + g)*VEC .. +VEC-1.
template <typename T, int R, bool KC>
__device__ __forceinline__ Frag<T> read_frag(const char* lds, int row, int ks, int g) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int PITCH = SlabLoader<T, R, KC>::PITCH;
  union {
    uint4 q;
    T e[VEC];
    Frag<T> f;
  } u;
  if (KC) {
    u.q = *reinterpret_cast<const uint4*>(lds + row * kRowPitchKC + (2 * ks + g) * 16);
  } else {
    const char* p = lds + (2 * ks + g) * VEC * PITCH + row * (int)sizeof(T);
#pragma unroll
    for (int e = 0; e < VEC; ++e) u.e[e] = *reinterpret_cast<const T*>(p + e * PITCH);
  }
  return u.f;
}

__device__ __forceinline__ void mma(const Frag<bf16_t>& a, const Frag<bf16_t>& b, f32x16& c) {
  c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}
__device__ __forceinline__ void mma(const Frag<float>& a, const Frag<float>& b, f32x16& c) {
  // Lane group g holds k = 4g+e in element e, so MFMA number e contracts k in {e, 4+e}.
#pragma unroll
  for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.f[e], b.f[e], c, 0, 0, 0);
}

template <typename T, int BM, int BN, bool AKC, bool BKC>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmArgs p) {
  using LA = SlabLoader<T, BM, AKC>;
  using LB = SlabLoader<T, BN, BKC>;
  constexpr int BK = LA::BK;
  constexpr int WM = BM / 2, WN = BN / 2, MT = WM / 32, NT = WN / 32;
  constexpr int STAGE = LA::BYTES + LB::BYTES;
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, g = lane >> 5;

  // Consecutive workgroup ids land on different XCDs (round robin over 8); give each XCD a
  // contiguous run of output tiles so its L2 sees neighbouring tiles that share operand rows.
  int bid = blockIdx.x;
  const int nb = p.tiles_m * p.tiles_n;
  if ((nb & 7) == 0) bid = (bid & 7) * (nb >> 3) + (bid >> 3);
  const int m0 = (bid / p.tiles_n) * BM;
  const int n0 = (bid % p.tiles_n) * BN;

  const long zo = blockIdx.y / p.zdiv, zi = blockIdx.y % p.zdiv;
  const T* A = reinterpret_cast<const T*>(p.a) + zo * p.a_so + zi * p.a_si;
  const T* B = reinterpret_cast<const T*>(p.b) + zo * p.b_so + zi * p.b_si;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  LA la;
  LB lb;
  const int nk = (p.k + BK - 1) / BK;
  if (nk > 0) {
    la.load(A, p.lda, m0, p.m, 0, p.k, p.vec_a, tid);
    lb.load(B, p.ldb, n0, p.n, 0, p.k, p.vec_b, tid);
    la.store(lds, tid);
    lb.store(lds + LA::BYTES, tid);
  }
  __syncthreads();

  for (int kt = 0; kt < nk; ++kt) {
    const char* sa = lds + (kt & 1) * STAGE;
    const char* sb = sa + LA::BYTES;
    const bool more = kt + 1 < nk;
    if (more) {
      la.load(A, p.lda, m0, p.m, (kt + 1) * BK, p.k, p.vec_a, tid);
      lb.load(B, p.ldb, n0, p.n, (kt + 1) * BK, p.k, p.vec_b, tid);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      Frag<T> fa[MT], fb[NT];
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[i] = read_frag<T, BM, AKC>(sa, wm * WM + i * 32 + li, ks, g);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[j] = read_frag<T, BN, BKC>(sb, wn * WN + j * 32 + li, ks, g);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) mma(fa[i], fb[j], acc[i][j]);
    }
    if (more) {
      char* da = lds + ((kt + 1) & 1) * STAGE;
      la.store(da, tid);
      lb.store(da + LA::BYTES, tid);
    }
    __syncthreads();
  }

  // Epilogue.  Accumulator register r of lane (li, g) is output row 8*(r/4) + 4*g + r%4, column li
  // of its 32x32 block.
  const bool out_f32 = p.flags & RTP_GEMM_OUT_F32;
  const bool cin_f32 = p.flags & RTP_GEMM_CIN_F32;
  const bool relu = p.flags & RTP_GEMM_RELU;
  char* cbase = p.c_out + (zo * p.c_so + zi * p.c_si) * (out_f32 ? 4 : (long)sizeof(T));
  const char* cin =
      p.c_in ? p.c_in + (zo * p.cin_so + zi * p.cin_si) * (cin_f32 ? 4 : (long)sizeof(T)) : nullptr;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + zo * p.bias_so + zi * p.bias_si : nullptr;
  const T* gate = p.gate ? reinterpret_cast<const T*>(p.gate) + zo * p.gate_so + zi * p.gate_si : nullptr;

#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int col = n0 + wn * WN + j * 32 + li;
      if (col >= p.n) continue;
      const float bv = bias ? to_f32(bias[col]) : 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (row >= p.m) continue;
        float v = p.alpha * acc[i][j][r];
        if (cin) {
          const long off = (long)row * p.ld_cin + col;
          v += cin_f32 ? reinterpret_cast<const float*>(cin)[off] : to_f32(reinterpret_cast<const T*>(cin)[off]);
        }
        v += bv;
        if (relu) v = fmaxf(v, 0.0f);
        if (gate) v = to_f32(gate[(long)row * p.ld_gate + col]) > 0.0f ? v : 0.0f;
        const long off = (long)row * p.ldc + col;
        if (out_f32)
          reinterpret_cast<float*>(cbase)[off] = v;
        else
          reinterpret_cast<T*>(cbase)[off] = from_f32<T>(v);
      }
    }
  }
}

template <typename T, int BM, int BN>
static int launch_layout(hipStream_t s, const GemmArgs& a, bool akc, bool bkc, dim3 grid) {
  if (akc && bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, true, true>), grid, dim3(kThreads), 0, s, a);
  else if (akc && !bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, true, false>), grid, dim3(kThreads), 0, s, a);
  else if (!akc && bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, false, true>), grid, dim3(kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, false, false>), grid, dim3(kThreads), 0, s, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

static bool mult(int64_t v, int64_t q) { return v % q == 0; }

template <typename T>
static int launch_gemm(hipStream_t s, const rtp_gemm_desc* d) {
  constexpr int VEC = 16 / sizeof(T);
  GemmArgs a;
  a.a = (const char*)d->a;
  a.b = (const char*)d->b;
  a.c_out = (char*)d->c_out;
  a.c_in = (const char*)d->c_in;
  a.bias = (const char*)d->bias;
  a.gate = (const char*)d->gate;
  a.m = (int)d->m;
  a.n = (int)d->n;
  a.k = (int)d->k;
  a.lda = d->lda;
  a.ldb = d->ldb;
  a.ldc = d->ldc;
  a.ld_cin = d->ld_cin;
  a.ld_gate = d->ld_gate;
  a.zdiv = (int)d->zdiv;
  a.a_so = d->a_so, a.a_si = d->a_si, a.b_so = d->b_so, a.b_si = d->b_si;
  a.c_so = d->c_so, a.c_si = d->c_si, a.cin_so = d->cin_so, a.cin_si = d->cin_si;
  a.gate_so = d->gate_so, a.gate_si = d->gate_si, a.bias_so = d->bias_so, a.bias_si = d->bias_si;
  a.alpha = d->alpha;
  a.flags = d->flags;
  a.vec_a = mult((int64_t)(uintptr_t)d->a, 16) && mult(d->lda, VEC) && mult(d->a_so, VEC) && mult(d->a_si, VEC);
  a.vec_b = mult((int64_t)(uintptr_t)d->b, 16) && mult(d->ldb, VEC) && mult(d->b_so, VEC) && mult(d->b_si, VEC);

  // Large tiles when they already fill the 256 CUs, small tiles otherwise.
  const int64_t big_tiles = ceil_div(d->m, 128) * ceil_div(d->n, 128) * d->batch;
  const bool big = big_tiles >= 192;
  const int bm = big ? 128 : 64;
  a.tiles_m = (int)ceil_div(d->m, bm);
  a.tiles_n = (int)ceil_div(d->n, bm);
  const int64_t nb = (int64_t)a.tiles_m * a.tiles_n;
  RTP_REQUIRE(nb < (1ll << 31) && d->batch < 65536, "gemm grid too large (%lld tiles, batch %lld)",
              (long long)nb, (long long)d->batch);
  dim3 grid((unsigned)nb, (unsigned)d->batch, 1);
  // variant name = the kernel template instance, e.g. gemm_bf16_64x64_kc_kc
  static const char* const names[2][2][2][2] = {
      {{{"gemm_f32_64x64_rc_rc", "gemm_f32_64x64_rc_kc"}, {"gemm_f32_64x64_kc_rc", "gemm_f32_64x64_kc_kc"}},
       {{"gemm_f32_128x128_rc_rc", "gemm_f32_128x128_rc_kc"}, {"gemm_f32_128x128_kc_rc", "gemm_f32_128x128_kc_kc"}}},
      {{{"gemm_bf16_64x64_rc_rc", "gemm_bf16_64x64_rc_kc"}, {"gemm_bf16_64x64_kc_rc", "gemm_bf16_64x64_kc_kc"}},
       {{"gemm_bf16_128x128_rc_rc", "gemm_bf16_128x128_rc_kc"},
        {"gemm_bf16_128x128_kc_rc", "gemm_bf16_128x128_kc_kc"}}}};
  const double mnk = (double)d->m * (double)d->n * (double)d->batch;
  const double out_sz = (d->flags & RTP_GEMM_OUT_F32) ? 4.0 : (double)sizeof(T);
  const double cin_sz = d->c_in ? ((d->flags & RTP_GEMM_CIN_F32) ? 4.0 : (double)sizeof(T)) : 0.0;
  const double bytes = ((double)d->m * d->k + (double)d->n * d->k) * d->batch * sizeof(T) + mnk * (out_sz + cin_sz);
  ProfileScope prof(s, names[sizeof(T) == 2][big][d->a_kcontig != 0][d->b_kcontig != 0], 2.0 * mnk * (double)d->k,
                    bytes);
  if (big) return launch_layout<T, 128, 128>(s, a, d->a_kcontig, d->b_kcontig, grid);
  return launch_layout<T, 64, 64>(s, a, d->a_kcontig, d->b_kcontig, grid);
}

// ---------------------------------------------------------------------------------------------
// Column sum (bias gradient): 64 columns per workgroup, 4 row phases, fixed-order reduction.
template <typename T>
__global__ __launch_bounds__(kThreads) void colsum_kernel(const T* x, long m, long n, long ld, void* out,
                                                          int out_f32, int accumulate) {
  __shared__ float part[4][64];
  const int c = threadIdx.x & 63, ph = threadIdx.x >> 6;
  const long col = (long)blockIdx.x * 64 + c;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < n) {
    long r = ph;
    for (; r + 12 < m; r += 16) {
      s0 += to_f32(x[r * ld + col]);
      s1 += to_f32(x[(r + 4) * ld + col]);
      s2 += to_f32(x[(r + 8) * ld + col]);
      s3 += to_f32(x[(r + 12) * ld + col]);
    }
    for (; r < m; r += 4) s0 += to_f32(x[r * ld + col]);
  }
  part[ph][c] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (ph == 0 && col < n) {
    float v = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
    if (out_f32) {
      float* o = reinterpret_cast<float*>(out);
      o[col] = accumulate ? o[col] + v : v;
    } else {
      T* o = reinterpret_cast<T*>(out);
      o[col] = from_f32<T>(accumulate ? to_f32(o[col]) + v : v);
    }
  }
}

}  // namespace rtp

extern "C" int rtp_gemm(void* stream, int dtype, const rtp_gemm_desc* d) {
  using namespace rtp;
  RTP_REQUIRE(d != nullptr, "rtp_gemm: null descriptor");
  RTP_REQUIRE(d->a && d->b && d->c_out, "rtp_gemm: null operand pointer");
  RTP_REQUIRE(d->m >= 0 && d->n >= 0 && d->k >= 0, "rtp_gemm: negative extent m=%lld n=%lld k=%lld",
              (long long)d->m, (long long)d->n, (long long)d->k);
  RTP_REQUIRE(d->m < (1ll << 31) && d->n < (1ll << 31) && d->k < (1ll << 31), "rtp_gemm: extent exceeds int32");
  RTP_REQUIRE(d->batch >= 1 && d->zdiv >= 1, "rtp_gemm: batch=%lld zdiv=%lld must be >= 1",
              (long long)d->batch, (long long)d->zdiv);
  RTP_REQUIRE(d->lda >= 1 && d->ldb >= 1 && d->ldc >= 1, "rtp_gemm: leading dimensions must be >= 1");
  RTP_REQUIRE(!d->c_in || d->ld_cin >= 1, "rtp_gemm: ld_cin must be >= 1 when c_in is given");
  RTP_REQUIRE(!d->gate || d->ld_gate >= 1, "rtp_gemm: ld_gate must be >= 1 when gate is given");
  if (d->m == 0 || d->n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RTP_F32) return launch_gemm<float>(s, d);
  if (dtype == RTP_BF16) return launch_gemm<bf16_t>(s, d);
  return fail(RTP_ERR_ARG, "rtp_gemm: unknown dtype %d", dtype);
}

extern "C" size_t rtp_gemm_desc_size(void) { return sizeof(rtp_gemm_desc); }

extern "C" int rtp_colsum(void* stream, int dtype, const void* x, int64_t m, int64_t n, int64_t ld, void* out,
                          int out_f32, int accumulate) {
  using namespace rtp;
  RTP_REQUIRE(x && out, "rtp_colsum: null pointer");
  RTP_REQUIRE(m >= 0 && n >= 0 && ld >= n, "rtp_colsum: bad shape m=%lld n=%lld ld=%lld", (long long)m,
              (long long)n, (long long)ld);
  if (n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)ceil_div(n, 64));
  ProfileScope prof(s, "colsum", (double)m * n, (double)m * n * (dtype == RTP_F32 ? 4 : 2));
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(colsum_kernel<float>, grid, dim3(kThreads), 0, s, (const float*)x, (long)m, (long)n,
                       (long)ld, out, 1, accumulate);
  else if (dtype == RTP_BF16)
    hipLaunchKernelGGL(colsum_kernel<bf16_t>, grid, dim3(kThreads), 0, s, (const bf16_t*)x, (long)m, (long)n,
                       (long)ld, out, out_f32, accumulate);
  else
    return fail(RTP_ERR_ARG, "rtp_colsum: unknown dtype %d", dtype);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
