// LDS-staged MFMA GEMM for gfx950 (fp32 via v_mfma_f32_32x32x2_f32, bf16 via v_mfma_f32_32x32x16_bf16)
// with the four operand layouts the rotated layers need (forward X W^T, input gradient dY W, weight
// gradient dY^T X, batched q k^T / p v), a fused epilogue (accumulate, bias, ReLU, ReLU-mask), and two
// ways of covering several rotation shards in ONE launch:
//   groups     : independent problems that differ only by a constant pointer stride per operand
//                (shard s of a column-parallel layer: W_s, b_s and the output column block s);
//   K segments : one output whose contraction runs over several shards in turn
//                (row-parallel outputs, input gradients of column-parallel layers: sum_s dY_s W_s),
//                accumulated in the MFMA accumulators, so the cross-shard sum never leaves registers.
//
// Work decomposition: 256 threads = 4 wavefronts in a 2x2 arrangement over a BM x BN output tile;
// each wavefront owns (BM/2)x(BN/2) as 32x32 MFMA blocks with fp32 accumulators in VGPRs.  The K loop
// moves 128-byte-per-row slabs (64 bf16 / 32 fp32 values of k) global -> registers -> LDS.  LDS is
// double buffered (one barrier per slab) and the global loads run DEPTH slabs ahead of the MFMAs in a
// ring of register buffers, which is what hides HBM/L2 latency when only one workgroup fits a CU.
#include "common.h"

#include <cstdlib>
#include <type_traits>

namespace rtp {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// Division of a 32-bit unsigned number by a launch constant with a multiply-high and two shifts (Granlund and
// Montgomery's round-up method, exact for every 32-bit dividend): integer division by a run-time value costs a
// few dozen dependent instructions on this hardware, and the wave-specialised kernel would otherwise do ten of
// them before it can issue its first load.
struct FastDiv {
  unsigned d, mul, s1, s2;
};
inline FastDiv make_fastdiv(unsigned d) {
  FastDiv f;
  f.d = d;
  unsigned s = 0;
  while ((1ull << s) < d) ++s;  // ceil(log2 d)
  f.mul = (unsigned)((((1ull << s) - d) << 32) / d + 1);
  f.s1 = s < 1 ? s : 1;
  f.s2 = s < 1 ? 0 : s - 1;
  return f;
}
__device__ __forceinline__ unsigned fast_div(unsigned n, const FastDiv& f) {
  const unsigned t = __umulhi(n, f.mul);
  return (t + ((n - t) >> f.s1)) >> f.s2;
}

struct GemmArgs {
  const char* a;
  const char* b;
  char* c_out;
  const char* c_in;
  const char* bias;
  const char* gate;
  int m, n, k, ksegs;
  long lda, ldb, ldc, ld_cin, ld_gate;
  int batch, zdiv;
  long a_so, a_si, b_so, b_si, c_so, c_si, cin_so, cin_si, gate_so, gate_si, bias_so, bias_si;
  long a_sg, b_sg, c_sg, cin_sg, gate_sg, bias_sg;
  long a_sk, b_sk, bias_sk;
  float alpha;
  int flags;
  int vec_a, vec_b;
  int tiles_m, tiles_n;
  int vec_c;       // every epilogue operand allows 16-byte accesses of 8 columns
  int xg, xm, xn;  // split of the (batch*groups, tiles_m, tiles_n) space over the 8 XCDs; xg == 0: none
  char* a_rowsum;  // bias gradient output (sum over k of A's rows), or null
  long rowsum_sg;
  // wave-specialised kernel: tile mapping without run-time divisions
  // A brick is mbk x nbk tiles; its tiles are handed out panel by panel, a panel being prow x pcol tiles with the
  // row running fastest, and the panels of a strip of pcol tile columns follow each other down the rows before
  // the next strip starts -- see the kernel.
  FastDiv d_batch, d_zdiv, d_tiles_n, d_brick, d_panel, d_prow, d_pm;  // divisors mbk*nbk, prow*pcol, prow, mbk/prow
  int mbk, nbk, prow, pcol;
  int xn_shift, xm_shift, zbk;  // log2 of xn and xm, batch*groups entries per brick
  unsigned long long* trace;    // null, or two words: earliest start / latest end of the launch on the wall clock
  float* sgd_master;            // null, or the fp32 parameters the product updates (indexed like c_out)
  char* sgd_w;                  // null, or the compute-dtype copy of the parameters
  float sgd_lr, sgd_clip;
  // softmax cross-entropy over the product's rows (the product is the logits of a column-parallel layer):
  // mode 1 leaves per-(row, 64-column block) {max, sum exp} and the target's logit instead of the logits,
  // mode 2 turns the logits into their gradient before they are stored
  int xent_mode, xent_blocks;   // blocks: 64-column blocks per row over all groups
  const long* xent_target;
  long xent_ignore;
  float2* xent_part;            // mode 1: [m][xent_blocks]
  float* xent_tlogit;           // mode 1: [m]
  const float2* xent_stats;     // mode 2: [m] {max, sum exp} of the whole row
  const float* xent_dloss;      // mode 2: upstream gradient, one scalar
  const float* xent_scale;      // mode 2: second scalar factor (1 / rows counted), or null
  // bytes that some later launch will read from HBM (the next layer's shards): requested here, see warm_ahead()
  const char* warm;
  long warm_bytes;
};

constexpr int kThreads = 256;
constexpr int kSlabBytes = 128;               // bytes of k per tile row and slab
constexpr int kRowPitchKC = kSlabBytes + 16;  // LDS row pitch when k is contiguous (16 B pad)

// Moves one R x BK operand slab global -> registers -> LDS.
//   KC  (k contiguous in memory): LDS holds [row][k], row pitch 144 bytes.
//   !KC (rows contiguous in memory): LDS holds [k][row], k pitch R*sizeof(T)+16 bytes.
template <typename T, int R, bool KC>
struct Slab {
  static constexpr int VEC = 16 / sizeof(T);
  static constexpr int BK = kSlabBytes / sizeof(T);
  static constexpr int KV = BK / VEC;           // 16-byte vectors per row (= 8)
  static constexpr int NV = R * KV / kThreads;  // vectors per thread
  static constexpr int RV = R / VEC;            // vectors per k line when rows are contiguous
  static constexpr int PITCH = KC ? kRowPitchKC : (R * (int)sizeof(T) + 16);
  static constexpr int BYTES = KC ? R * kRowPitchKC : BK * PITCH;
  uint4 reg[NV];

  // FAST: every 16-byte vector of the slab is either wholly inside the operand or wholly outside it
  // (guaranteed by the host: aligned pointers and strides, extents that are multiples of VEC), so a
  // vector is loaded unconditionally from a clamped address; vectors beyond the contraction length are
  // replaced by zeros later, when the registers are moved to LDS (store with ktail), so nothing here
  // consumes a load result and all loads of a slab stay in flight.  Rows beyond the operand are clamped
  // too: they only feed accumulators the epilogue never stores.
  // !FAST: element-wise guarded loads for ragged or unaligned operands.
  template <bool FAST>
  __device__ __forceinline__ void load(const T* base, long ld, int row0, int rows, int k0, int kdim, int tid) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * kThreads;
      union {
        uint4 q;
        T e[VEC];
      } u;
      if (KC) {
        const int row = row0 + v / KV;
        const int k = k0 + (v % KV) * VEC;
        if (FAST) {
          const int rc = row < rows ? row : rows - 1;
          const int kc = k < kdim ? k : 0;
          u.q = *reinterpret_cast<const uint4*>(base + (long)rc * ld + kc);
        } else {
          const T* src = base + (long)row * ld + k;
#pragma unroll
          for (int e = 0; e < VEC; ++e) u.e[e] = (row < rows && k + e < kdim) ? src[e] : (T)0.0f;
        }
      } else {
        const int k = k0 + v / RV;
        const int row = row0 + (v % RV) * VEC;
        if (FAST) {
          const int kc = k < kdim ? k : 0;
          const int rc = row < rows ? row : 0;
          u.q = *reinterpret_cast<const uint4*>(base + (long)kc * ld + rc);
        } else {
          const T* src = base + (long)k * ld + row;
#pragma unroll
          for (int e = 0; e < VEC; ++e) u.e[e] = (k < kdim && row + e < rows) ? src[e] : (T)0.0f;
        }
      }
      reg[i] = u.q;
    }
  }

  // ktail: the slab that starts at k0 reaches beyond kdim, zero the vectors that lie outside.
  __device__ __forceinline__ void store(char* lds, int tid, bool ktail, int k0, int kdim) const {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int v = tid + i * kThreads;
      char* dst = KC ? lds + (v / KV) * kRowPitchKC + (v % KV) * 16 : lds + (v / RV) * PITCH + (v % RV) * 16;
      uint4 q = reg[i];
      if (ktail) {
        const int k = KC ? k0 + (v % KV) * VEC : k0 + v / RV;
        const bool live = k < kdim;
        q.x = live ? q.x : 0u;
        q.y = live ? q.y : 0u;
        q.z = live ? q.z : 0u;
        q.w = live ? q.w : 0u;
      }
      *reinterpret_cast<uint4*>(dst) = q;
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
  constexpr int PITCH = Slab<T, R, KC>::PITCH;
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

// Sum of the fragment's k values in fp32 (the lane's share of a row sum of A).
__device__ __forceinline__ float frag_sum(const Frag<bf16_t>& a, float s) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const bf16x2 pr = {a.v[2 * e], a.v[2 * e + 1]};
    s = __builtin_amdgcn_fdot2_f32_bf16(pr, one, s, false);
  }
  return s;
}
__device__ __forceinline__ float frag_sum(const Frag<float>& a, float s) {
  return s + ((a.f[0] + a.f[1]) + (a.f[2] + a.f[3]));
}

// Fused epilogue shared by the GEMM kernels.  Accumulator register r of lane (li, g) is output row
// 8*(r/4) + 4*g + r%4, column li of its 32x32 block.
template <typename T, int MT, int NT, int WM, int WN>
__device__ __forceinline__ void store_tile(const GemmArgs& p, f32x16 (&acc)[MT][NT], int m0, int n0, int wm, int wn,
                                           int li, int g, int grp, long zo, long zi) {
  const bool out_f32 = p.flags & RTP_GEMM_OUT_F32;
  const bool cin_f32 = p.flags & RTP_GEMM_CIN_F32;
  const bool relu = p.flags & RTP_GEMM_RELU;
  char* cbase = p.c_out + (grp * p.c_sg + zo * p.c_so + zi * p.c_si) * (out_f32 ? 4 : (long)sizeof(T));
  const char* cin =
      p.c_in ? p.c_in + (grp * p.cin_sg + zo * p.cin_so + zi * p.cin_si) * (cin_f32 ? 4 : (long)sizeof(T)) : nullptr;
  const T* bias =
      p.bias ? reinterpret_cast<const T*>(p.bias) + grp * p.bias_sg + zo * p.bias_so + zi * p.bias_si : nullptr;
  const T* gate =
      p.gate ? reinterpret_cast<const T*>(p.gate) + grp * p.gate_sg + zo * p.gate_so + zi * p.gate_si : nullptr;

#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int col = n0 + wn * WN + j * 32 + li;
      if (col >= p.n) continue;
      float bv = 0.0f;
      if (bias) {
        // a bias per K segment (row-parallel shards each carry bias/ws): summed in segment order
        const int nb_seg = p.bias_sk ? p.ksegs : 1;
        for (int sgm = 0; sgm < nb_seg; ++sgm) bv += to_f32(bias[sgm * p.bias_sk + col]);
      }
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

template <typename T, int BM, int BN, bool AKC, bool BKC, int DEPTH, bool FAST>
struct GemmTile {
  using LA = Slab<T, BM, AKC>;
  using LB = Slab<T, BN, BKC>;
  static constexpr int BK = LA::BK;
  static constexpr int WM = BM / 2, WN = BN / 2, MT = WM / 32, NT = WN / 32;
  static constexpr int STAGE = LA::BYTES + LB::BYTES;
  static constexpr int KSTEPS = 4;  // slab k extent / (2*VEC)

  const GemmArgs& p;
  const T* A;
  const T* B;
  int m0, n0, tid, nk_seg;
  LA la[DEPTH];
  LB lb[DEPTH];

  __device__ __forceinline__ GemmTile(const GemmArgs& args) : p(args) {}

  template <int R>
  __device__ __forceinline__ void fetch(int slab) {
    const int seg = slab / nk_seg;
    const int k0 = (slab - seg * nk_seg) * BK;
    la[R].template load<FAST>(A + seg * p.a_sk, p.lda, m0, p.m, k0, p.k, tid);
    lb[R].template load<FAST>(B + seg * p.b_sk, p.ldb, n0, p.n, k0, p.k, tid);
  }
  // `slab` is the slab held by register slot R; only the last slab of a K segment can be partial.
  template <int R>
  __device__ __forceinline__ void stash(char* stage, int slab) {
    const int seg = slab / nk_seg;
    const int k0 = (slab - seg * nk_seg) * BK;
    const bool ktail = FAST && k0 + BK > p.k;
    la[R].store(stage, tid, ktail, k0, p.k);
    lb[R].store(stage + LA::BYTES, tid, ktail, k0, p.k);
  }
};

template <typename T, int BM, int BN, bool AKC, bool BKC, int DEPTH, bool FAST>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmArgs p) {
  using G = GemmTile<T, BM, BN, AKC, BKC, DEPTH, FAST>;
  constexpr int MT = G::MT, NT = G::NT, WM = G::WM, WN = G::WN, STAGE = G::STAGE;
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

  const int grp = blockIdx.y / p.batch, zb = blockIdx.y % p.batch;
  const long zo = zb / p.zdiv, zi = zb % p.zdiv;

  G t(p);
  t.tid = tid;
  t.m0 = (bid / p.tiles_n) * BM;
  t.n0 = (bid % p.tiles_n) * BN;
  t.A = reinterpret_cast<const T*>(p.a) + grp * p.a_sg + zo * p.a_so + zi * p.a_si;
  t.B = reinterpret_cast<const T*>(p.b) + grp * p.b_sg + zo * p.b_so + zi * p.b_si;
  t.nk_seg = (p.k + G::BK - 1) / G::BK;
  const int nk = t.nk_seg * p.ksegs;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Prologue: slabs 0..DEPTH-1 into the register ring, slab 0 on into LDS stage 0.
  if (nk > 0) t.template fetch<0>(0);
  if (DEPTH > 1 && nk > 1) t.template fetch<1 % DEPTH>(1);
  if (DEPTH > 2 && nk > 2) t.template fetch<2 % DEPTH>(2);
  if (nk > 0) t.template stash<0>(lds, 0);
  __syncthreads();

  auto compute = [&](int kt) {
    const char* sa = lds + (kt & 1) * STAGE;
    const char* sb = sa + G::LA::BYTES;
#pragma unroll
    for (int ks = 0; ks < G::KSTEPS; ++ks) {
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
  };

  // Steady state for slab kt (register slot kt % DEPTH was just emptied into LDS): refill that slot
  // with slab kt+DEPTH, run the MFMAs of slab kt from LDS stage kt&1, move slab kt+1 from its register
  // slot to the other LDS stage, barrier.  While 2*DEPTH slabs remain none of this needs a guard, so the
  // loop body is branch-free and the loads of DEPTH slabs stay in flight across the barriers.
  int kt = 0;
  for (; kt + 2 * DEPTH <= nk; kt += DEPTH) {
    t.template fetch<0>(kt + DEPTH);
    compute(kt);
    t.template stash<1 % DEPTH>(lds + ((kt + 1) & 1) * STAGE, kt + 1);
    __syncthreads();
    if (DEPTH > 1) {
      t.template fetch<1 % DEPTH>(kt + 1 + DEPTH);
      compute(kt + 1);
      t.template stash<2 % DEPTH>(lds + ((kt + 2) & 1) * STAGE, kt + 2);
      __syncthreads();
    }
    if (DEPTH > 2) {
      t.template fetch<2 % DEPTH>(kt + 2 + DEPTH);
      compute(kt + 2);
      t.template stash<0>(lds + ((kt + 3) & 1) * STAGE, kt + 3);
      __syncthreads();
    }
  }
  // Drain: the same phases with guards (kt is a multiple of DEPTH, so the slot assignment continues).
  for (; kt < nk; kt += DEPTH) {
    if (kt + DEPTH < nk) t.template fetch<0>(kt + DEPTH);
    compute(kt);
    if (kt + 1 < nk) t.template stash<1 % DEPTH>(lds + ((kt + 1) & 1) * STAGE, kt + 1);
    __syncthreads();
    if (DEPTH > 1) {
      if (kt + 1 >= nk) break;
      if (kt + 1 + DEPTH < nk) t.template fetch<1 % DEPTH>(kt + 1 + DEPTH);
      compute(kt + 1);
      if (kt + 2 < nk) t.template stash<2 % DEPTH>(lds + ((kt + 2) & 1) * STAGE, kt + 2);
      __syncthreads();
    }
    if (DEPTH > 2) {
      if (kt + 2 >= nk) break;
      if (kt + 2 + DEPTH < nk) t.template fetch<2 % DEPTH>(kt + 2 + DEPTH);
      compute(kt + 2);
      if (kt + 3 < nk) t.template stash<0>(lds + ((kt + 3) & 1) * STAGE, kt + 3);
      __syncthreads();
    }
  }

  store_tile<T, MT, NT, WM, WN>(p, acc, t.m0, t.n0, wm, wn, li, g, grp, zo, zi);
}

// Epilogue of the direct-to-LDS kernel.  `ct` is the BM x BN tile of raw accumulators in LDS (row pitch BN+4
// floats).  Thread `tid` of NTHR finishes chunks of 8 consecutive columns: alpha * acc (+ c_in) (+ bias) -> ReLU ->
// gate mask -> store, the same order of operations as store_tile.  With p.vec_c (16-byte aligned operands and
// n % 8 == 0, checked by the host) every global access of a chunk is a 16-byte vector.
template <typename T>
__device__ __forceinline__ void load8(const T* src, float (&v)[8]) {
  if (sizeof(T) == 2) {
    union {
      uint4 q;
      T e[8];
    } u;
    u.q = *reinterpret_cast<const uint4*>(src);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f32(u.e[e]);
  } else {
    const float4 lo = reinterpret_cast<const float4*>(src)[0], hi = reinterpret_cast<const float4*>(src)[1];
    v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
  }
}
template <typename T>
__device__ __forceinline__ void store8(T* dst, const float (&v)[8], bool stream) {
  if (sizeof(T) == 2) {
    union {
      uint4 q;
      T e[8];
    } u;
#pragma unroll
    for (int e = 0; e < 8; ++e) u.e[e] = from_f32<T>(v[e]);
    if (stream)
      nt_store(u.q, reinterpret_cast<uint4*>(dst));
    else
      *reinterpret_cast<uint4*>(dst) = u.q;
  } else if (stream) {
    nt_store(make_float4(v[0], v[1], v[2], v[3]), reinterpret_cast<float4*>(dst));
    nt_store(make_float4(v[4], v[5], v[6], v[7]), reinterpret_cast<float4*>(dst) + 1);
  } else {
    reinterpret_cast<float4*>(dst)[0] = make_float4(v[0], v[1], v[2], v[3]);
    reinterpret_cast<float4*>(dst)[1] = make_float4(v[4], v[5], v[6], v[7]);
  }
}

// Raw 16-byte-vector image of 8 consecutive epilogue operand values (c_in in `dtype` or fp32, bias, gate): what a thread
// requests for all of its chunks before it consumes any of them.
template <typename T>
struct Raw8 {
  uint4 q[sizeof(T) == 2 ? 1 : 2];
  __device__ __forceinline__ void load(const T* src) {
    q[0] = reinterpret_cast<const uint4*>(src)[0];
    if (sizeof(T) == 4) q[sizeof(T) == 2 ? 0 : 1] = reinterpret_cast<const uint4*>(src)[1];
  }
  __device__ __forceinline__ void get(float (&v)[8]) const {
    if (sizeof(T) == 2) {
      union {
        uint4 q;
        T e[8];
      } u;
      u.q = q[0];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = to_f32(u.e[e]);
    } else {
      union {
        uint4 q[2];
        float f[8];
      } u;
      u.q[0] = q[0], u.q[1] = q[sizeof(T) == 2 ? 0 : 1];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = u.f[e];
    }
  }
};

template <typename T, int BM, int BN, int NTHR>
__device__ __forceinline__ void finish_tile(const GemmArgs& p, const float* ct, int m0, int n0, int tid, int grp,
                                            long zo, long zi) {
  constexpr int CP = BN + 4, CPR = BN / 8, CHUNKS = BM * CPR;
  const bool stream_out = p.flags & RTP_GEMM_STREAM_OUT;
  const bool out_f32 = p.flags & RTP_GEMM_OUT_F32;
  const bool cin_f32 = p.flags & RTP_GEMM_CIN_F32;
  const bool relu = p.flags & RTP_GEMM_RELU;
  char* cbase = p.c_out + (grp * p.c_sg + zo * p.c_so + zi * p.c_si) * (out_f32 ? 4 : (long)sizeof(T));
  const char* cin =
      p.c_in ? p.c_in + (grp * p.cin_sg + zo * p.cin_so + zi * p.cin_si) * (cin_f32 ? 4 : (long)sizeof(T)) : nullptr;
  const T* bias =
      p.bias ? reinterpret_cast<const T*>(p.bias) + grp * p.bias_sg + zo * p.bias_so + zi * p.bias_si : nullptr;
  const T* gate =
      p.gate ? reinterpret_cast<const T*>(p.gate) + grp * p.gate_sg + zo * p.gate_so + zi * p.gate_si : nullptr;
  const int nb_seg = p.bias_sk ? p.ksegs : 1;  // a bias per K segment is summed in segment order
  const long zoff = grp * p.c_sg + zo * p.c_so + zi * p.c_si;
  float* master = p.sgd_master ? p.sgd_master + zoff : nullptr;
  T* wcopy = p.sgd_w ? reinterpret_cast<T*>(p.sgd_w) + zoff : nullptr;
  const bool skip_out = p.flags & RTP_GEMM_SGD_SKIP_OUT;

  if constexpr (CHUNKS % NTHR == 0) {
    // The common form (vector-aligned operands, one bias vector): a thread requests the bias, the addend and the mask
    // of ALL its chunks before it consumes the first -- one trip to memory for the whole epilogue instead of one per
    // chunk (a store to c_out may alias a later chunk's c_in as far as the compiler knows, so left alone the loads of
    // chunk i + 1 wait behind the store of chunk i).  When the thread count is a multiple of the chunks per row all of
    // a thread's chunks lie in the same 8 columns and share one bias vector.
    if (p.vec_c && nb_seg == 1 && p.xent_mode == 0 && master == nullptr) {
      constexpr int NCH = CHUNKS / NTHR;
      constexpr bool SAMECOL = NTHR % CPR == 0;
      constexpr int NB = SAMECOL ? 1 : NCH;
      Raw8<T> rb[NB], rg[NCH], rc16[NCH];
      Raw8<float> rc32[NCH];
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = tid + i * NTHR;
        const int row = m0 + c / CPR, col = n0 + (c % CPR) * 8;
        const int colc = col < p.n ? col : 0;
        const long rowc = row < p.m ? row : p.m - 1;
        if (bias && (i == 0 || !SAMECOL)) rb[SAMECOL ? 0 : i].load(bias + colc);
        if (cin) {
          if (cin_f32)
            rc32[i].load(reinterpret_cast<const float*>(cin) + rowc * p.ld_cin + colc);
          else
            rc16[i].load(reinterpret_cast<const T*>(cin) + rowc * p.ld_cin + colc);
        }
        if (gate) rg[i].load(gate + rowc * p.ld_gate + colc);
      }
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        const int c = tid + i * NTHR;
        const int lr = c / CPR, lc = (c % CPR) * 8;
        const int row = m0 + lr, col = n0 + lc;
        const bool col_ok = col < p.n;
        float v[8], t[8];
        const float4 lo = *reinterpret_cast<const float4*>(ct + lr * CP + lc);
        const float4 hi = *reinterpret_cast<const float4*>(ct + lr * CP + lc + 4);
        v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= p.alpha;
        if (cin) {
          if (cin_f32)
            rc32[i].get(t);
          else
            rc16[i].get(t);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += t[e];
        }
        if (bias) {
          rb[SAMECOL ? 0 : i].get(t);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += t[e];
        }
        if (relu) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = fmaxf(v[e], 0.0f);
        }
        if (gate) {
          rg[i].get(t);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = t[e] > 0.0f ? v[e] : 0.0f;
        }
        if (row >= p.m || !col_ok) continue;
        const long off = (long)row * p.ldc + col;
        if (out_f32)
          store8(reinterpret_cast<float*>(cbase) + off, v, stream_out);
        else
          store8(reinterpret_cast<T*>(cbase) + off, v, stream_out);
      }
      return;
    }
  }

  for (int c = tid; c < CHUNKS; c += NTHR) {
    const int lr = c / CPR, lc = (c % CPR) * 8;
    const int row = m0 + lr, col = n0 + lc;
    if (row >= p.m || col >= p.n) continue;
    float v[8], t[8];
    {
      const float4 lo = *reinterpret_cast<const float4*>(ct + lr * CP + lc);
      const float4 hi = *reinterpret_cast<const float4*>(ct + lr * CP + lc + 4);
      v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= p.alpha;
    if (p.vec_c) {
      if (cin) {
        const long off = (long)row * p.ld_cin + col;
        if (cin_f32)
          load8(reinterpret_cast<const float*>(cin) + off, t);
        else
          load8(reinterpret_cast<const T*>(cin) + off, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
      }
      if (bias) {
        // The per-segment biases of a row-parallel layer sit in eight different home rows, far from any cache: the
        // loads of eight segments are issued together (segments past the last re-read segment 0 and count as zero)
        // and then added in segment order -- one trip to memory instead of one per segment.
        float bv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int s0 = 0; s0 < nb_seg; s0 += 8) {
          float bt[8][8];
#pragma unroll
          for (int j = 0; j < 8; ++j) load8(bias + (s0 + j < nb_seg ? s0 + j : 0) * p.bias_sk + col, bt[j]);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float on = s0 + j < nb_seg ? 1.0f : 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) bv[e] += on * bt[j][e];
          }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += bv[e];
      }
      if (relu) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = fmaxf(v[e], 0.0f);
      }
      if (gate) {
        load8(gate + (long)row * p.ld_gate + col, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = t[e] > 0.0f ? v[e] : 0.0f;
      }
      if (p.xent_mode == 2) {
        // logits -> their cross-entropy gradient: (softmax - onehot(target)) * dloss (* scale); rows whose target
        // is the ignore index or outside the classes get zeros
        const long tg = p.xent_target[row];
        const bool live = tg != p.xent_ignore && tg >= 0 && tg < (long)p.xent_blocks * 64;
        const float2 st = p.xent_stats[row];
        const float inv = 1.0f / st.y;
        const float sc = live ? p.xent_dloss[0] * (p.xent_scale ? p.xent_scale[0] : 1.0f) : 0.0f;
        const long gcol = (long)grp * p.n + col;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float gq = expf(to_f32(from_f32<T>(v[e])) - st.x) * inv;
          if (gcol + e == tg) gq -= 1.0f;
          v[e] = gq * sc;
        }
      }
      const long off = (long)row * p.ldc + col;
      if (master) {
        float w[8];
        load8(master + off, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = sgd_update<T>(w[e], v[e], p.sgd_lr, p.sgd_clip);
        store8(master + off, w, true);
        if (wcopy) store8(wcopy + off, w, true);
      }
      if (!skip_out) {
        if (out_f32)
          store8(reinterpret_cast<float*>(cbase) + off, v, stream_out);
        else
          store8(reinterpret_cast<T*>(cbase) + off, v, stream_out);
      }
    } else {
      for (int e = 0; e < 8 && col + e < p.n; ++e) {
        float x = v[e];
        if (cin) {
          const long off = (long)row * p.ld_cin + col + e;
          x += cin_f32 ? reinterpret_cast<const float*>(cin)[off] : to_f32(reinterpret_cast<const T*>(cin)[off]);
        }
        if (bias) {
          float bv = 0.0f;
          for (int sgm = 0; sgm < nb_seg; ++sgm) bv += to_f32(bias[sgm * p.bias_sk + col + e]);
          x += bv;
        }
        if (relu) x = fmaxf(x, 0.0f);
        if (gate) x = to_f32(gate[(long)row * p.ld_gate + col + e]) > 0.0f ? x : 0.0f;
        const long off = (long)row * p.ldc + col + e;
        if (master) {
          const float w = sgd_update<T>(master[off], x, p.sgd_lr, p.sgd_clip);
          master[off] = w;
          if (wcopy) wcopy[off] = from_f32<T>(w);
        }
        if (skip_out) continue;
        if (out_f32)
          reinterpret_cast<float*>(cbase)[off] = x;
        else
          reinterpret_cast<T*>(cbase)[off] = from_f32<T>(x);
      }
    }
  }
}

// Epilogue of a logits product whose rows only feed a softmax cross-entropy (mode 1): thread r of the first BM
// threads walks row r of the tile in LDS, 64 columns at a time, and leaves {max, sum exp(v - max)} of every
// 64-column block in part[row][block] -- the block index runs over the layer's whole output row, group after
// group, so the layout does not depend on the tile shape -- and the logit of the row's target where this tile
// holds it.  The logits themselves are not stored.  v = alpha * acc + bias, rounded to T as the stored logits would
// be, so that loss and gradient are those of the logits a separate product would have written.
template <typename T, int BM, int BN, int NTHR>
__device__ __forceinline__ void finish_tile_xent_stats(const GemmArgs& p, const float* ct, int m0, int n0, int tid,
                                                       int grp) {
  static_assert(BN % 64 == 0 && BM <= NTHR, "64-column blocks, one thread per tile row");
  constexpr int CP = BN + 4;
  if (tid >= BM) return;
  const int row = m0 + tid;
  if (row >= p.m) return;
  const T* bias = p.bias ? reinterpret_cast<const T*>(p.bias) + grp * p.bias_sg : nullptr;
  const long t = p.xent_target[row];
  const long tcol = t - (long)grp * p.n;  // the target's column inside this group, if it is in [0, n)
  const float* crow = ct + tid * CP;
#pragma unroll
  for (int b = 0; b < BN / 64; ++b) {
    const int col0 = n0 + b * 64;
    if (col0 >= p.n) break;
    float mx = -INFINITY;
    for (int j = 0; j < 64; ++j) {
      float v = p.alpha * crow[b * 64 + j];
      if (bias) v += to_f32(bias[col0 + j]);
      v = to_f32(from_f32<T>(v));
      mx = fmaxf(mx, v);
      if (col0 + j == tcol) p.xent_tlogit[row] = v;
    }
    float sum = 0.0f;
    for (int j = 0; j < 64; ++j) {
      float v = p.alpha * crow[b * 64 + j];
      if (bias) v += to_f32(bias[col0 + j]);
      v = to_f32(from_f32<T>(v));
      sum += expf(v - mx);
    }
    p.xent_part[(long)row * p.xent_blocks + ((long)grp * p.n + col0) / 64] = make_float2(mx, sum);
  }
}

// Epilogue of a product whose result is consumed by the fused clip + SGD update (a weight gradient: no c_in, bias,
// ReLU or mask; 16-byte aligned operands, checked by the host).  The fp32 parameters of up to four of the thread's
// chunks are requested before the first of them is needed, so the trips to memory overlap instead of following
// each other; rows / columns outside the problem read a clamped address and store nothing.
template <typename T, int BM, int BN, int NTHR>
__device__ __forceinline__ void finish_tile_sgd(const GemmArgs& p, const float* ct, int m0, int n0, int tid, int grp,
                                                long zo, long zi) {
  constexpr int CP = BN + 4, CPR = BN / 8, CHUNKS = BM * CPR, NCH = CHUNKS / NTHR;
  constexpr int BATCH = NCH % 4 == 0 ? 4 : (NCH % 3 == 0 ? 3 : (NCH % 2 == 0 ? 2 : 1));
  static_assert(CHUNKS % NTHR == 0 && NCH % BATCH == 0, "every thread owns the same number of chunks");
  const bool stream_out = p.flags & RTP_GEMM_STREAM_OUT;
  const bool skip_out = p.flags & RTP_GEMM_SGD_SKIP_OUT;
  const long zoff = grp * p.c_sg + zo * p.c_so + zi * p.c_si;
  T* cbase = reinterpret_cast<T*>(p.c_out) + zoff;
  float* master = p.sgd_master + zoff;
  T* wcopy = p.sgd_w ? reinterpret_cast<T*>(p.sgd_w) + zoff : nullptr;
#pragma unroll
  for (int b0 = 0; b0 < NCH; b0 += BATCH) {
    float w[BATCH][8];
    long off[BATCH];
    bool live[BATCH];
#pragma unroll
    for (int i = 0; i < BATCH; ++i) {
      const int c = tid + (b0 + i) * NTHR;
      const int row = m0 + c / CPR, col = n0 + (c % CPR) * 8;
      live[i] = row < p.m && col < p.n;
      off[i] = (long)(row < p.m ? row : p.m - 1) * p.ldc + (col < p.n ? col : 0);
      load8(master + off[i], w[i]);
    }
#pragma unroll
    for (int i = 0; i < BATCH; ++i) {
      const int c = tid + (b0 + i) * NTHR;
      const int lr = c / CPR, lc = (c % CPR) * 8;
      float v[8];
      const float4 lo = *reinterpret_cast<const float4*>(ct + lr * CP + lc);
      const float4 hi = *reinterpret_cast<const float4*>(ct + lr * CP + lc + 4);
      v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[e] *= p.alpha;
        w[i][e] = sgd_update<T>(w[i][e], v[e], p.sgd_lr, p.sgd_clip);
      }
      if (!live[i]) continue;
      store8(master + off[i], w[i], true);
      if (wcopy) store8(wcopy + off[i], w[i], true);
      if (!skip_out) store8(cbase + off[i], v, stream_out);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Direct-to-LDS pipeline (the fast path).  Slabs go global -> LDS with global_load_lds_dwordx4: no
// staging registers, NSTAGE LDS stages, up to NSTAGE-1 slabs in flight while the MFMAs of the current slab
// run.  The compiler does not order these asynchronous LDS writes against later LDS reads, so the kernel
// does it by hand: in the middle of the phase of slab k every wave waits until its own loads of slab k+1
// have landed (s_waitcnt vmcnt(N), loads retire in order) and then meets the workgroup barrier; after the
// barrier slab k+1 may be read, and the stage of slab k-1 (whose fragments every wave consumed in its
// previous phase) is refilled.
//
// A wave-level load writes 64 lanes x 16 B = 1 KiB of consecutive LDS, so rows cannot be padded.  For a
// k-contiguous operand (LDS [row][128 B]) bank conflicts are avoided by an XOR swizzle instead: the
// 16-byte chunk c of row r is kept at chunk position c ^ (r & 7); the lane that fills position cp of row
// r fetches chunk cp ^ (r & 7) from global memory.  A row-contiguous operand is kept as [k][rows].
// Vectors beyond the contraction length are fetched from a 16-byte block of zeros; rows beyond the
// operand are clamped (they only feed accumulators that are never stored).
//
// The workgroup has 8 waves with separate roles: waves 0..3 run the MFMAs of a 2x2 grid of wave tiles and
// issue no global loads; waves 4..7 only issue the loads and count them down.  Scalar bookkeeping for the
// loads therefore does not take issue slots from the MFMA waves.
__device__ __attribute__((aligned(16))) unsigned int g_zero16[4] = {0u, 0u, 0u, 0u};

// s_waitcnt with vmcnt = VM, lgkmcnt = 0, expcnt untouched (gfx9 encoding).
#define RTP_WAIT_VM_LGKM0(VM) __builtin_amdgcn_s_waitcnt(((VM)&0xF) | (((VM) >> 4) << 14) | (0x7 << 4))
// s_waitcnt with vmcnt = VM only (expcnt and lgkmcnt untouched).
#define RTP_WAIT_VM(VM) __builtin_amdgcn_s_waitcnt(((VM)&0xF) | (((VM) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// LDS has 64 four-byte banks (256 bytes per clock).  Swizzles keep the lanes that are served in one clock on
// different banks:
//  * k-contiguous operand, [row][128 B]: 16 consecutive rows read the same 16-byte chunk c; row r keeps it at
//    chunk position c ^ ((r >> 1) & 7), which together with the row's parity (rows alternate between the two
//    128-byte halves of the bank space) gives 16 different 16-byte bank slots.
//  * row-contiguous 16-bit operand, [k][rows]: a transposing read touches 4 consecutive k lines x 64 bytes; the
//    chunk index inside k line kl is XORed with rc_swizzle(kl) so that the 4 lines fall on different slots.
template <typename T, int R>
__device__ __forceinline__ constexpr int rc_swizzle(int kl) {
  if (sizeof(T) != 2) return 0;
  return R >= 128 ? (kl & 3) << 2 : ((kl >> 1) & 1) << 2;
}

// Chunk swizzle of a k-contiguous operand whose slab rows are SB bytes (128: 8 chunks, 64: 4 chunks): 16
// consecutive rows reading the same chunk must land on 16 different 16-byte slots of the 256-byte bank space.
template <int SB>
__device__ __forceinline__ constexpr int kc_swizzle(int row) {
  return SB == 128 ? (row >> 1) & 7 : (row >> 2) & 3;
}

template <typename T, int R, bool KC, int NL, int SB>
struct DmaOperand {
  static constexpr int VEC = 16 / sizeof(T);
  static_assert(SB == 128 || SB == 64, "slab rows of 128 or 64 bytes");
  static_assert((R * SB / 1024) % NL == 0, "every loader wave issues the same number of loads");
  static constexpr int NI = R * SB / 1024 / NL;   // load instructions (1 KiB each) per loader wave and slab
  static constexpr int BYTES = R * SB;            // one stage of this operand
  static constexpr int LINE = R * (int)sizeof(T); // bytes of one k line when rows are contiguous
  static_assert(KC || 1024 % LINE == 0 || LINE % 1024 == 0, "a 1 KiB load covers whole k lines or a whole fraction of one");
  // The lane's vector sits at `ofs` bytes from the slab's base pointer, which is the same for every lane and lives
  // in scalar registers: the loader's steady state then has no vector-ALU instruction at all.  (A vector add per
  // load has to compete for issue slots with the MFMAs of the compute wave on the same SIMD, and loses: measured,
  // per-lane 64-bit pointers make the loads of a slab take the MFMA time longer.)
  unsigned ofs[NI];
  int koff[NI];  // k of the vector inside its slab

  // Base pointer of the first slab: row row0 of a K-contiguous operand, element row0 of k line 0 otherwise.
  __device__ __forceinline__ static const char* slab_base(const T* x, long ld, int row0) {
    return reinterpret_cast<const char*>(KC ? x + (long)row0 * ld : x + row0);
  }

  // lw: index of the loader wave (0..NL-1).  The host guarantees that a tile's offsets fit 32 bits.
  __device__ __forceinline__ void init(long ld, int row0, int rows, int lw, int lane) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int j = lw * NI + i;  // which KiB of the stage
      if (KC) {
        constexpr int LPR = SB / 16;  // lanes (16-byte chunks) per row
        const int row = j * (64 / LPR) + lane / LPR;
        const int c = (lane % LPR) ^ kc_swizzle<SB>(row);
        const int rr = row0 + row < rows ? row : rows - 1 - row0;  // rows past the end re-read the last one
        ofs[i] = (unsigned)((long)rr * ld * (long)sizeof(T)) + (unsigned)(c * 16);
        koff[i] = c * VEC;
      } else {
        const int byte = lane * 16;
        const int kl = j * (1024 / LINE) + byte / LINE;
        int chunk = ((byte % LINE) >> 4) ^ rc_swizzle<T, R>(kl);  // which 16 bytes of the k line land here
        if (row0 + chunk * VEC + VEC > rows) chunk = 0;           // past the end: re-read the tile's first rows
        ofs[i] = (unsigned)((long)kl * ld * (long)sizeof(T)) + (unsigned)(chunk * 16);
        koff[i] = kl;
      }
    }
  }

  // Start the loads of the slab at `base` into the stage at LDS byte address `lds_stage` (this operand's part).
  // TAIL: the slab is the last of its K segment (first k = k0) and reaches beyond the contraction length kdim;
  // vectors beyond it come from a block of zeros (per-lane addresses, the one case that needs them).
  template <bool TAIL>
  __device__ __forceinline__ void issue(unsigned lds_stage, int lw, const char* base, int k0, int kdim) const {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      // Inline assembly on purpose: the compiler must not track this instruction (it would make LDS reads wait
      // for all outstanding loads); the kernel's explicit s_waitcnt + barrier protocol is the ordering that counts.
      if (TAIL) {
        const char* src = base + ofs[i];
        if (k0 + koff[i] >= kdim) src = reinterpret_cast<const char*>(g_zero16);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :
                     : "s"(lds_stage + (unsigned)((lw * NI + i) * 1024)), "v"(src)
                     : "memory");
      } else {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_stage + (unsigned)((lw * NI + i) * 1024)), "v"(ofs[i]), "s"(base)
                     : "memory");
      }
    }
  }
};

// The next layer's shards arrive while this product computes.  Weights are read once per pass, so at their turn
// they come from HBM, whose latency the NSTAGE - 1 slabs in flight do not cover: measured on the LM's shapes, a
// product takes 15 - 30 % longer on weights from HBM than on weights that sit in the 256 MiB memory-side cache.
// So a product can be handed the bytes that the *next* products will need: its MFMA waves, idle until the first
// slab has landed, request them right at kernel start, 1 KiB per instruction, straight into 1 KiB of LDS that
// nothing reads (no registers, and nobody ever waits for these loads: an MFMA wave next waits for vector memory
// in the epilogue).  Pieces are dealt round-robin over (workgroup, wave), so the launch as a whole reads the region
// front to back; a wave asks for at most kWarmMax pieces (the counter of outstanding loads has 6 bits), the rest
// of a larger region stays unread.
constexpr int kWarmMax = 48;
__device__ __forceinline__ void warm_ahead(const GemmArgs& p, unsigned lds_dst, unsigned wg, unsigned nwg, int wave,
                                           int lane) {
  if (p.warm == nullptr) return;
  const long pieces = p.warm_bytes >> 10;
  long piece = (long)wg * 4 + wave;
  for (int j = 0; j < kWarmMax && piece < pieces; ++j, piece += (long)nwg * 4) {
    const char* src = p.warm + (piece << 10) + lane * 16;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_dst), "v"(src) : "memory");
  }
}

typedef short short4_t __attribute__((ext_vector_type(4)));

// rowbase: first tile row of the 32-row MFMA block; the lane's own row is rowbase + lane % 32.
template <typename T, int R, bool KC, int SB>
__device__ __forceinline__ Frag<T> read_frag_dma(const char* st, int rowbase, int lane, int ks) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int LINE = R * (int)sizeof(T);
  const int li = lane & 31, g = lane >> 5;
  union {
    uint4 q;
    T e[VEC];
    short4_t h[2];
    Frag<T> f;
  } u;
  if (KC) {
    const int row = rowbase + li;
    u.q = *reinterpret_cast<const uint4*>(st + row * SB + (((2 * ks + g) ^ kc_swizzle<SB>(row)) << 4));
  } else if (sizeof(T) == 2) {
    // LDS holds [k][rows] (rows contiguous) but the MFMA wants 8 consecutive k per lane.  gfx950's
    // transposing LDS read does the 16-bit transpose inside each group of 16 lanes: lane s of a group
    // supplies the address of 4 consecutive rows at k line (s / 4); the group then receives, in lane j,
    // the 4 consecutive k of row (4 * (s % 4) ... ) + j.  Two such reads give the 8 k of the lane's row.
    const int s16 = lane & 15, blk = (lane >> 4) & 1;
    const int kl = (2 * ks + g) * 8 + (s16 >> 2);         // k line of the first read; the second is kl + 4
    const int rb = (rowbase + 16 * blk + 4 * (s16 & 3)) * 2;  // byte of the lane's 4 rows inside the k line
    const int c0 = (rb >> 4) ^ rc_swizzle<T, R>(kl), c1 = (rb >> 4) ^ rc_swizzle<T, R>(kl + 4);
    const char* p0 = st + kl * LINE + (c0 << 4) + (rb & 15);
    const char* p1 = st + (kl + 4) * LINE + (c1 << 4) + (rb & 15);
    u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p0));
    u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(p1));
  } else {
    const char* p = st + (2 * ks + g) * VEC * LINE + (rowbase + li) * (int)sizeof(T);
#pragma unroll
    for (int e = 0; e < VEC; ++e) u.e[e] = *reinterpret_cast<const T*>(p + e * LINE);
  }
  return u.f;
}

// The body of the product kernel: workgroup `id` of the `nwg` that work on the problem `p` (`bx`, `by`: its
// coordinates in a launch that does not use XCD bricks).  `p` lives in the kernel-argument segment.
template <typename T, int BM, int BN, bool AKC, bool BKC, int NSTAGE, int SB, int PD>
__device__ __forceinline__ void gemm_dma_body(const GemmArgs& p, const unsigned id, const unsigned bx, const unsigned by,
                                              const unsigned nwg) {
  constexpr int NL = 4;  // loader waves (waves 4..7); waves 0..3 compute
  using DA = DmaOperand<T, BM, AKC, NL, SB>;
  using DB = DmaOperand<T, BN, BKC, NL, SB>;
  constexpr int BK = SB / sizeof(T);
  constexpr int KS = SB / 32;  // MFMA k-steps per slab
  // the four MFMA waves form a 2 x 2 grid of wave tiles, or 4 x 1 where half the tile's columns are no whole number
  // of 32-column MFMA blocks (BN = 160)
  constexpr int WGM = (BN / 2) % 32 == 0 ? 2 : 4, WGN = 4 / WGM;
  constexpr int WM = BM / WGM, WN = BN / WGN, MT = WM / 32, NT = WN / 32;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tiles are whole 32 x 32 MFMA blocks");
  constexpr int STAGE = DA::BYTES + DB::BYTES;
  constexpr int NI = DA::NI + DB::NI;  // loads per loader wave and slab
  static_assert((NSTAGE - 2) * NI < 64, "vmcnt is a 6-bit counter");
  static_assert(NSTAGE >= 3, "at least 3 LDS stages");
  static_assert(NSTAGE * STAGE + 1024 <= 160 * 1024, "160 KiB of LDS per workgroup");
  static_assert(BM * (BN + 4) * 4 <= NSTAGE * STAGE, "the epilogue stages the fp32 tile in the slab memory");
  // Stage addresses are compile-time offsets into one array, so LDS reads carry immediate offsets.  The last KiB
  // is where the loads of warm_ahead() land.
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE + 1024];

  const int tid = threadIdx.x;
  unsigned long long t_start = 0, t_ready = 0, t_loop = 0;  // phase stamps of thread 0 (an MFMA wave), mode 2 only
  if (p.trace != nullptr && tid == 0) {
    t_start = (unsigned long long)wall_clock64();
    atomicMin(p.trace, t_start);
  }
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = WGM == 2 ? (wave >> 1) & 1 : wave & 3, wn = WGM == 2 ? wave & 1 : 0;
  const int li = lane & 31, g = lane >> 5;

  // Workgroups are handed to the 8 XCDs round-robin in launch order, and every XCD has its own L2.  The
  // host splits the (batch*groups, tiles_m, tiles_n) space into 8 bricks (xg * xm * xn == 8) chosen so that
  // the operand rows one XCD touches are as few as possible; workgroup `id` works on brick id % 8.
  // Both mappings are computed and one is selected, without a branch: every kernel argument is then fetched by
  // one batch of scalar loads at entry instead of three dependent rounds (each a trip to memory on a cold cache).
  const unsigned xcd = id & 7, slot = id >> 3;
  // The ~32 workgroups an XCD runs at a time should cover a compact block of the brick, not a row of it: they
  // share the XCD's L2, and a 4 x 8 block of tiles reads 12 tile-operands where a 1 x 32 row reads 33.  Over the
  // rounds of a long launch the panels walk down a strip of pcol tile columns, whose B operand stays in the L2
  // while the A rows stream past once per strip.
  const unsigned zl = fast_div(slot, p.d_brick);  // entry of the batch*groups axis inside the brick
  const unsigned t = slot - zl * p.d_brick.d;      // tile inside the mbk x nbk brick
  const unsigned q = fast_div(t, p.d_panel), r = t - q * p.d_panel.d;  // panel, tile inside the panel
  const unsigned cn = fast_div(r, p.d_prow), cm = r - cn * p.d_prow.d;
  const unsigned qn = fast_div(q, p.d_pm), qm = q - qn * p.d_pm.d;     // strip, panel inside the strip
  const int tile_n_x = (int)((xcd & ((1u << p.xn_shift) - 1)) * p.nbk + qn * p.pcol + cn);
  const int tile_m_x = (int)(((xcd >> p.xn_shift) & ((1u << p.xm_shift) - 1)) * p.mbk + qm * p.prow + cm);
  const int z_x = (int)((xcd >> (p.xn_shift + p.xm_shift)) * p.zbk + zl);
  const int tile_m_p = (int)fast_div(bx, p.d_tiles_n);
  const int tile_n_p = (int)(bx - tile_m_p * p.d_tiles_n.d);
  const bool bricks = p.xg != 0;
  const int tile_m = bricks ? tile_m_x : tile_m_p, tile_n = bricks ? tile_n_x : tile_n_p;
  const int z = bricks ? z_x : (int)by;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;
  const int grp = (int)fast_div(z, p.d_batch), zb = z - grp * (int)p.d_batch.d;
  const long zo = fast_div(zb, p.d_zdiv), zi = zb - (int)zo * (int)p.d_zdiv.d;
  const int nk_seg = (p.k + BK - 1) / BK;
  const int nk = nk_seg * p.ksegs;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  float rsum[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) rsum[i] = 0.0f;

  // Barrier protocol: both paths meet the same nk barriers.  Barrier k is passed when slab k is visible to
  // every wave: a loader reaches it only after its own loads of slab k have landed.  A compute wave reaches
  // barrier k+1 after the MFMAs that consumed the last fragments of slab k-1, so once barrier k+1 is passed
  // the loaders may refill the stage of slab k-1 (with slab k-1+NSTAGE).
  if (wave >= 4) {
    // ---- loader waves: issue slabs strictly in order, NSTAGE-1 ahead of the slab being consumed ----
    const int lw = wave - 4;
    const T* A = reinterpret_cast<const T*>(p.a) + grp * p.a_sg + zo * p.a_so + zi * p.a_si;
    const T* B = reinterpret_cast<const T*>(p.b) + grp * p.b_sg + zo * p.b_so + zi * p.b_si;
    DA da;
    DB db;
    da.init(p.lda, m0, p.m, lw, lane);
    db.init(p.ldb, n0, p.n, lw, lane);
    const char* ca = DA::slab_base(A, p.lda, m0);  // base of the next slab, uniform: scalar registers
    const char* cb = DB::slab_base(B, p.ldb, n0);
    constexpr long SZ = (long)sizeof(T);
    const long step_a = (AKC ? (long)BK : (long)BK * p.lda) * SZ, step_b = (BKC ? (long)BK : (long)BK * p.ldb) * SZ;
    // after the last slab of a segment the pointers move to the start of the next segment
    const long last_a = step_a + p.a_sk * SZ - nk_seg * step_a, last_b = step_b + p.b_sk * SZ - nk_seg * step_b;
    const int k0_last = (nk_seg - 1) * BK;
    const bool tail = p.k % BK != 0;
    const unsigned lds0 = (unsigned)(uintptr_t)(lptr_t)lds;
    unsigned fill = lds0;  // LDS address of the stage the next slab goes to
    int left = nk_seg;     // slabs left in the current K segment, the next one included
    auto issue = [&]() {
      if (left != 1 || !tail) {
        da.template issue<false>(fill, lw, ca, 0, 0);
        db.template issue<false>(fill + DA::BYTES, lw, cb, 0, 0);
      } else {
        da.template issue<true>(fill, lw, ca, k0_last, p.k);
        db.template issue<true>(fill + DA::BYTES, lw, cb, k0_last, p.k);
      }
      if (left != 1) {
        ca += step_a;
        cb += step_b;
        --left;
      } else {
        ca += last_a;
        cb += last_b;
        left = nk_seg;
      }
      fill += STAGE;
      if (fill == lds0 + NSTAGE * STAGE) fill = lds0;
    };
    const int ahead = nk < NSTAGE - 1 ? nk : NSTAGE - 1;
    for (int s_ = 0; s_ < ahead; ++s_) issue();
    if (nk >= NSTAGE - 1) {
      RTP_WAIT_VM((NSTAGE - 2) * NI);
    } else {
      RTP_WAIT_VM(0);
    }
    __builtin_amdgcn_s_barrier();  // barrier 0
    int k = 0;
    for (; k + NSTAGE - 1 < nk; ++k) {  // slab k+NSTAGE-1 exists: steady state
      RTP_WAIT_VM((NSTAGE - 3) * NI);   // slabs k+2 .. k+NSTAGE-2 may still be in flight
      __builtin_amdgcn_s_barrier();     // barrier k+1
      issue();                          // slab k+NSTAGE-1 into the stage of slab k-1
    }
    for (; k + 1 < nk; ++k) {
      RTP_WAIT_VM(0);
      __builtin_amdgcn_s_barrier();
    }
  } else {
    // ---- compute waves ----
    // Software pipeline over k-steps (KS per slab, numbered through the slabs): the fragments of k-step t + PD are
    // read from LDS right before the MFMAs of k-step t are issued, into one of PD + 1 register sets.  A wave gets
    // one 16-byte LDS read back every ~16 clocks after ~130-200 clocks of latency, so a read needs several k-steps
    // of MFMAs (32 clocks each) to hide behind; PD is chosen per tile shape for that.  The barrier that makes slab
    // k+1 visible sits right before its first fragment read, i.e. PD k-steps before its first MFMA.
    constexpr int NSET = PD + 1;
    static_assert(PD >= 1 && PD <= KS, "prefetch distance of 1..KS k-steps");
    static_assert((NSTAGE * KS) % NSET == 0, "register set of a k-step must not depend on the round");
    Frag<T> fa[NSET][MT], fb[NSET][NT];
    // Row sums of A (a bias gradient) ride along in the waves of the tile row's first tile that own column
    // block 0: each lane adds up the k values of its own row as the fragments pass by.
    const bool rowsum = p.a_rowsum != nullptr && tile_n == 0 && wn == 0;
    auto read_step = [&](auto S, auto Q, auto SET) {
      const char* sa = lds + (decltype(S)::value % NSTAGE) * STAGE;
      const char* sb = sa + DA::BYTES;
      constexpr int q = decltype(Q)::value, set = decltype(SET)::value;
#pragma unroll
      for (int i = 0; i < MT; ++i) fa[set][i] = read_frag_dma<T, BM, AKC, SB>(sa, wm * WM + i * 32, lane, q);
#pragma unroll
      for (int j = 0; j < NT; ++j) fb[set][j] = read_frag_dma<T, BN, BKC, SB>(sb, wn * WN + j * 32, lane, q);
    };
    auto mma_step = [&](auto SET) {
      constexpr int set = decltype(SET)::value;
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j) mma(fa[set][i], fb[set][j], acc[i][j]);
      if (rowsum) {
#pragma unroll
        for (int i = 0; i < MT; ++i) rsum[i] = frag_sum(fa[set][i], rsum[i]);
      }
    };
    // k-step Q of slab k (stage S).  The scheduling fences keep the order written here: left alone, the compiler
    // sinks every LDS read to just before the MFMA that uses it (fewest live registers), which puts the LDS
    // latency in front of each MFMA instead of behind earlier ones.
    auto step = [&](auto S, auto Q, int k, auto STEADY) {
      constexpr bool steady = decltype(STEADY)::value;
      constexpr int s = decltype(S)::value, q = decltype(Q)::value;
      constexpr int t = s * KS + q;                            // k-step number inside the round
      constexpr int tq = (q + PD) % KS, ds = (q + PD) / KS;    // the k-step to prefetch: tq of slab k + ds
      if (steady || k + ds < nk) {
        if (ds == 1 && tq == 0) {
          __builtin_amdgcn_s_barrier();  // barrier k+1: slab k+1 is visible
          __builtin_amdgcn_sched_barrier(0);
        }
        read_step(std::integral_constant<int, (s + ds) % NSTAGE>{}, std::integral_constant<int, tq>{},
                  std::integral_constant<int, (t + PD) % NSET>{});
      }
      mma_step(std::integral_constant<int, t % NSET>{});
      // Issue order inside the step: one MFMA, then its share of the step's LDS reads, and so on.  A wave issues in
      // order and an MFMA holds the issue port until the matrix pipe takes it, so only what sits between two
      // MFMAs is issued in an MFMA's shadow; reads bunched up before the first MFMA would leave the pipe idle.
      constexpr int RPF_A = AKC ? 1 : (sizeof(T) == 2 ? 2 : 4), RPF_B = BKC ? 1 : (sizeof(T) == 2 ? 2 : 4);
      constexpr int NR = MT * RPF_A + NT * RPF_B, NM = MT * NT * (sizeof(T) == 2 ? 1 : 4);
      constexpr int PER = (NR + NM - 1) / NM;
      [&]<int... I>(std::integer_sequence<int, I...>) {
        ((__builtin_amdgcn_sched_group_barrier(0x008, 1, 0),
          (I * PER < NR ? __builtin_amdgcn_sched_group_barrier(0x100, (I + 1) * PER <= NR ? PER : NR - I * PER, 0)
                        : (void)0)),
         ...);
      }(std::make_integer_sequence<int, NM>{});
      __builtin_amdgcn_sched_barrier(0);
    };
    auto phase = [&](auto S, int k, auto STEADY) {
      if (!decltype(STEADY)::value && k >= nk) return;
      [&]<int... Q>(std::integer_sequence<int, Q...>) {
        (step(S, std::integral_constant<int, Q>{}, k, STEADY), ...);
      }(std::make_integer_sequence<int, KS>{});
    };
    // one round = NSTAGE phases with compile-time stage indices
    auto round = [&](int kt, auto STEADY) {
      [&]<int... S>(std::integer_sequence<int, S...>) {
        (phase(std::integral_constant<int, S>{}, kt + S, STEADY), ...);
      }(std::make_integer_sequence<int, NSTAGE>{});
    };
    warm_ahead(p, (unsigned)(uintptr_t)(lptr_t)lds + NSTAGE * STAGE, id, nwg, wave, lane);
    if (p.bias != nullptr && wave == 0) {
      // the epilogue's bias values (one vector per K segment of a row-parallel layer, each in another home row) are
      // requested now and sit in the L2 when the epilogue asks for them
      const int nb = p.bias_sk ? p.ksegs : 1;
      const T* bs = reinterpret_cast<const T*>(p.bias) + grp * p.bias_sg + zo * p.bias_so + zi * p.bias_si + n0;
      constexpr int LPS = (BN * (int)sizeof(T) + 63) / 64;  // lanes per segment: one per 64 bytes of the tile's columns
      const int sgm = lane / LPS, part = lane % LPS;
      if (sgm < nb && n0 + part * (64 / (int)sizeof(T)) + 4 / (int)sizeof(T) <= p.n) {  // the 4 bytes read lie inside the vector
        const char* src = reinterpret_cast<const char*>(bs + (long)sgm * p.bias_sk) + part * 64;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                     :
                     : "s"((unsigned)(uintptr_t)(lptr_t)lds + NSTAGE * STAGE), "v"(src)
                     : "memory");
      }
    }
    if (p.gate != nullptr && p.vec_c) {
      // the ReLU mask of the epilogue is an activation saved by the forward pass, long gone from the caches: the
      // tile's part of it is requested now, 16 bytes per lane
      constexpr int CPR = BN * (int)sizeof(T) / 16, NCH = BM * CPR;  // 16-byte chunks per tile row, per tile
      const T* gt = reinterpret_cast<const T*>(p.gate) + grp * p.gate_sg + zo * p.gate_so + zi * p.gate_si;
#pragma unroll
      for (int c0 = 0; c0 < NCH; c0 += 256) {
        const int c = c0 + wave * 64 + lane;
        const int row = m0 + c / CPR, col = n0 + (c % CPR) * (16 / (int)sizeof(T));
        if (c < NCH && row < p.m && col + 16 / (int)sizeof(T) <= p.n) {
          const char* src = reinterpret_cast<const char*>(gt + (long)row * p.ld_gate + col);
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                       :
                       : "s"((unsigned)(uintptr_t)(lptr_t)lds + NSTAGE * STAGE), "v"(src)
                       : "memory");
        }
      }
    }
    __builtin_amdgcn_s_barrier();  // barrier 0
    if (p.trace != nullptr && tid == 0) t_ready = (unsigned long long)wall_clock64();
    [&]<int... Q>(std::integer_sequence<int, Q...>) {
      (read_step(std::integral_constant<int, 0>{}, std::integral_constant<int, Q>{}, std::integral_constant<int, Q>{}),
       ...);
    }(std::make_integer_sequence<int, PD>{});
    __builtin_amdgcn_sched_barrier(0);
    int kt = 0;
    for (; kt + NSTAGE < nk; kt += NSTAGE) round(kt, std::true_type{});
    for (; kt < nk; kt += NSTAGE) round(kt, std::false_type{});
    if (p.trace != nullptr && tid == 0) t_loop = (unsigned long long)wall_clock64();
  }
  const bool computes = wave < 4;
  if (computes && p.a_rowsum != nullptr && tile_n == 0 && wn == 0) {
    // lanes 0..31 and 32..63 hold the two k halves of the same 32 rows
    T* dst = reinterpret_cast<T*>(p.a_rowsum) + grp * p.rowsum_sg;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const float v = rsum[i] + __shfl_xor(rsum[i], 32, 64);
      const int row = m0 + wm * WM + i * 32 + li;
      if (g == 0 && row < p.m) dst[row] = from_f32<T>((p.flags & RTP_GEMM_ROWSUM_ACCUM) ? to_f32(dst[row]) + v : v);
    }
  }

  // Epilogue through LDS: the accumulators (fp32) are laid out as the BM x BN tile, then every thread of the
  // workgroup, loader waves included, finishes 8 consecutive columns of one row and writes them with 16-byte
  // stores.
  __builtin_amdgcn_s_barrier();  // every wave has read its last fragments
  constexpr int CP = BN + 4;     // row pitch in floats
  float* ct = reinterpret_cast<float*>(lds);
  if (computes) {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          ct[(wm * WM + i * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * CP + wn * WN + j * 32 + li] = acc[i][j][r];
  }
  __syncthreads();
  if (p.sgd_master != nullptr && p.vec_c)
    finish_tile_sgd<T, BM, BN, 512>(p, ct, m0, n0, tid, grp, zo, zi);
  else if (p.xent_mode == 1) {
    // (tiles whose width is no multiple of the 64-column statistics blocks are never chosen for this epilogue)
    if constexpr (BN % 64 == 0) finish_tile_xent_stats<T, BM, BN, 512>(p, ct, m0, n0, tid, grp);
  } else
    finish_tile<T, BM, BN, 512>(p, ct, m0, n0, tid, grp, zo, zi);
  if (p.trace != nullptr && tid == 0) {
    const unsigned long long t_end = (unsigned long long)wall_clock64();
    atomicMax(p.trace + 1, t_end);
    // the phase sums come from every 16th workgroup: atomics of all of them on one line would stretch the launch
    if ((id & 15u) != 0u) return;
    atomicAdd(p.trace + 2, t_start);
    atomicAdd(p.trace + 3, t_ready - t_start);
    atomicAdd(p.trace + 4, t_loop - t_ready);
    atomicAdd(p.trace + 5, t_end - t_loop);
    atomicAdd(p.trace + 6, 1ull);
  }
}

template <typename T, int BM, int BN, bool AKC, bool BKC, int NSTAGE, int SB, int PD>
__global__ __launch_bounds__(512) void gemm_dma_kernel(GemmArgs p) {
  touch_kernel_arguments<sizeof(GemmArgs)>();
  gemm_dma_body<T, BM, BN, AKC, BKC, NSTAGE, SB, PD>(p, blockIdx.x + blockIdx.y * gridDim.x, blockIdx.x, blockIdx.y,
                                                     gridDim.x * gridDim.y);
}

// ---------------------------------------------------------------------------------------------
// 256 x 256 tiles for large products.  What bounds the kernel above on a large product is the stream of operand
// bytes from the L2 into the LDS (a product of 4096^3 takes as long with its MFMAs removed), and that stream is
// (1/BM + 1/BN) bytes per flop: a 256 x 256 tile moves two thirds of what 256 x 128 moves.  Its 256 KiB of fp32
// accumulators need all eight waves of the workgroup as MFMA waves (2 x 4 wave tiles of 128 x 64, 128 accumulator
// registers each), so here the waves issue the direct-to-LDS loads themselves, each an eighth of a slab, right
// after the barrier that frees a stage.  Both roles in one wave allow a tighter stage protocol than above: every
// read of slab k's fragments is issued before the first read of slab k+1, and the barrier of slab k+1 sits in front
// of that read -- so once a wave has seen its own LDS reads return (lgkmcnt 0) and has passed barrier k+1, nobody
// reads the stage of slab k any more and slab k + NSTAGE may go there.  NSTAGE slabs are in LDS or on their way;
// the k-step being multiplied lives in registers.  With NSTAGE = 2 this is the plain double buffer, and the two
// stages can hold slabs of 128 bytes of k per row (2 x 64 KiB): a load instruction then fetches whole cache lines
// of a K-contiguous operand (with 64-byte rows its operand stream alone took 1.5 x as long as that of a
// row-contiguous operand), and a barrier comes every 4 k-steps.  The epilogue goes through LDS in four passes of
// 64 rows.
template <typename T, bool AKC, bool BKC, int NSTAGE, int SB, int PD>
__global__ __launch_bounds__(512) void gemm_dma8_kernel(GemmArgs p) {
  constexpr int BM = 256, BN = 256, NL = 8;
  using DA = DmaOperand<T, BM, AKC, NL, SB>;
  using DB = DmaOperand<T, BN, BKC, NL, SB>;
  constexpr int BK = SB / sizeof(T);
  constexpr int KS = SB / 32;
  constexpr int WM = 128, WN = 64, MT = 4, NT = 2;
  constexpr int STAGE = DA::BYTES + DB::BYTES;
  constexpr int NI = DA::NI + DB::NI;
  static_assert((NSTAGE - 1) * NI < 64, "vmcnt is a 6-bit counter");
  static_assert(NSTAGE >= 2 && NSTAGE * STAGE <= 160 * 1024, "2 or more stages within 160 KiB of LDS");
  static_assert(64 * (BN + 4) * 4 <= NSTAGE * STAGE, "an epilogue pass stages 64 rows of the fp32 tile");
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];

  touch_kernel_arguments<sizeof(GemmArgs)>();
  const int tid = threadIdx.x;
  if (p.trace != nullptr && tid == 0) atomicMin(p.trace, (unsigned long long)wall_clock64());
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int li = lane & 31, g = lane >> 5;

  // tile mapping: as in gemm_dma_kernel
  const unsigned id = blockIdx.x + blockIdx.y * gridDim.x;
  const unsigned xcd = id & 7, slot = id >> 3;
  const unsigned zl = fast_div(slot, p.d_brick);
  const unsigned t_ = slot - zl * p.d_brick.d;
  const unsigned q_ = fast_div(t_, p.d_panel), r_ = t_ - q_ * p.d_panel.d;
  const unsigned cn = fast_div(r_, p.d_prow), cm = r_ - cn * p.d_prow.d;
  const unsigned qn = fast_div(q_, p.d_pm), qm = q_ - qn * p.d_pm.d;
  const int tile_n_x = (int)((xcd & ((1u << p.xn_shift) - 1)) * p.nbk + qn * p.pcol + cn);
  const int tile_m_x = (int)(((xcd >> p.xn_shift) & ((1u << p.xm_shift) - 1)) * p.mbk + qm * p.prow + cm);
  const int z_x = (int)((xcd >> (p.xn_shift + p.xm_shift)) * p.zbk + zl);
  const int tile_m_p = (int)fast_div(blockIdx.x, p.d_tiles_n);
  const int tile_n_p = (int)(blockIdx.x - tile_m_p * p.d_tiles_n.d);
  const bool bricks = p.xg != 0;
  const int tile_m = bricks ? tile_m_x : tile_m_p, tile_n = bricks ? tile_n_x : tile_n_p;
  const int z = bricks ? z_x : (int)blockIdx.y;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;
  const int grp = (int)fast_div(z, p.d_batch), zb = z - grp * (int)p.d_batch.d;
  const long zo = fast_div(zb, p.d_zdiv), zi = zb - (int)zo * (int)p.d_zdiv.d;
  const int nk_seg = (p.k + BK - 1) / BK;
  const int nk = nk_seg * p.ksegs;

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  float rsum[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) rsum[i] = 0.0f;

  // ---- this wave's share of the loads ----
  const T* A = reinterpret_cast<const T*>(p.a) + grp * p.a_sg + zo * p.a_so + zi * p.a_si;
  const T* B = reinterpret_cast<const T*>(p.b) + grp * p.b_sg + zo * p.b_so + zi * p.b_si;
  DA da;
  DB db;
  da.init(p.lda, m0, p.m, wave, lane);
  db.init(p.ldb, n0, p.n, wave, lane);
  const char* ca = DA::slab_base(A, p.lda, m0);
  const char* cb = DB::slab_base(B, p.ldb, n0);
  constexpr long SZ = (long)sizeof(T);
  const long step_a = (AKC ? (long)BK : (long)BK * p.lda) * SZ, step_b = (BKC ? (long)BK : (long)BK * p.ldb) * SZ;
  const long last_a = step_a + p.a_sk * SZ - nk_seg * step_a, last_b = step_b + p.b_sk * SZ - nk_seg * step_b;
  const int k0_last = (nk_seg - 1) * BK;
  const bool tail = p.k % BK != 0;
  const unsigned lds0 = (unsigned)(uintptr_t)(lptr_t)lds;
  unsigned fill = lds0;
  int left = nk_seg;
  auto issue = [&]() {
    if (left != 1 || !tail) {
      da.template issue<false>(fill, wave, ca, 0, 0);
      db.template issue<false>(fill + DA::BYTES, wave, cb, 0, 0);
    } else {
      da.template issue<true>(fill, wave, ca, k0_last, p.k);
      db.template issue<true>(fill + DA::BYTES, wave, cb, k0_last, p.k);
    }
    if (left != 1) {
      ca += step_a;
      cb += step_b;
      --left;
    } else {
      ca += last_a;
      cb += last_b;
      left = nk_seg;
    }
    fill += STAGE;
    if (fill == lds0 + NSTAGE * STAGE) fill = lds0;
  };

  constexpr int NSET = PD + 1;
  static_assert(PD >= 1 && PD <= KS, "prefetch distance of 1..KS k-steps");
  static_assert((NSTAGE * KS) % NSET == 0, "register set of a k-step must not depend on the round");
  Frag<T> fa[NSET][MT], fb[NSET][NT];
  const bool rowsum = p.a_rowsum != nullptr && tile_n == 0 && wn == 0;
  auto read_step = [&](auto S, auto Q, auto SET) {
    const char* sa = lds + (decltype(S)::value % NSTAGE) * STAGE;
    const char* sb = sa + DA::BYTES;
    constexpr int q = decltype(Q)::value, set = decltype(SET)::value;
#pragma unroll
    for (int i = 0; i < MT; ++i) fa[set][i] = read_frag_dma<T, BM, AKC, SB>(sa, wm * WM + i * 32, lane, q);
#pragma unroll
    for (int j = 0; j < NT; ++j) fb[set][j] = read_frag_dma<T, BN, BKC, SB>(sb, wn * WN + j * 32, lane, q);
  };
  auto mma_step = [&](auto SET) {
    constexpr int set = decltype(SET)::value;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) mma(fa[set][i], fb[set][j], acc[i][j]);
    if (rowsum) {
#pragma unroll
      for (int i = 0; i < MT; ++i) rsum[i] = frag_sum(fa[set][i], rsum[i]);
    }
  };
  auto step = [&](auto S, auto Q, int k, auto STEADY) {
    constexpr bool steady = decltype(STEADY)::value;
    constexpr int s = decltype(S)::value, q = decltype(Q)::value;
    constexpr int t = s * KS + q;
    constexpr int tq = (q + PD) % KS, ds = (q + PD) / KS;
    if (steady || k + ds < nk) {
      if (ds == 1 && tq == 0) {
        // barrier k+1: my loads of slab k+1 have landed (those of the slabs up to k+NSTAGE-1 may be on their way)
        // and my reads of slab k have returned; behind it that holds for everybody, and the stage of slab k takes
        // slab k+NSTAGE
        if (k + NSTAGE - 1 < nk) {
          RTP_WAIT_VM_LGKM0((NSTAGE - 2) * NI);
        } else {
          RTP_WAIT_VM_LGKM0(0);
        }
        __builtin_amdgcn_s_barrier();
        if (k + NSTAGE < nk) issue();
        __builtin_amdgcn_sched_barrier(0);
      }
      read_step(std::integral_constant<int, (s + ds) % NSTAGE>{}, std::integral_constant<int, tq>{},
                std::integral_constant<int, (t + PD) % NSET>{});
    }
    mma_step(std::integral_constant<int, t % NSET>{});
    constexpr int RPF_A = AKC ? 1 : (sizeof(T) == 2 ? 2 : 4), RPF_B = BKC ? 1 : (sizeof(T) == 2 ? 2 : 4);
    constexpr int NR = MT * RPF_A + NT * RPF_B, NM = MT * NT * (sizeof(T) == 2 ? 1 : 4);
    constexpr int PER = (NR + NM - 1) / NM;
    [&]<int... I>(std::integer_sequence<int, I...>) {
      ((__builtin_amdgcn_sched_group_barrier(0x008, 1, 0),
        (I * PER < NR ? __builtin_amdgcn_sched_group_barrier(0x100, (I + 1) * PER <= NR ? PER : NR - I * PER, 0)
                      : (void)0)),
       ...);
    }(std::make_integer_sequence<int, NM>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  auto phase = [&](auto S, int k, auto STEADY) {
    if (!decltype(STEADY)::value && k >= nk) return;
    [&]<int... Q>(std::integer_sequence<int, Q...>) {
      (step(S, std::integral_constant<int, Q>{}, k, STEADY), ...);
    }(std::make_integer_sequence<int, KS>{});
  };
  auto round = [&](int kt, auto STEADY) {
    [&]<int... S>(std::integer_sequence<int, S...>) {
      (phase(std::integral_constant<int, S>{}, kt + S, STEADY), ...);
    }(std::make_integer_sequence<int, NSTAGE>{});
  };

  // prologue: NSTAGE slabs on their way, slab 0 landed
  const int ahead = nk < NSTAGE ? nk : NSTAGE;
  for (int s_ = 0; s_ < ahead; ++s_) issue();
  if (nk >= NSTAGE) {
    RTP_WAIT_VM((NSTAGE - 1) * NI);
  } else {
    RTP_WAIT_VM(0);
  }
  __builtin_amdgcn_s_barrier();  // barrier 0
  [&]<int... Q>(std::integer_sequence<int, Q...>) {
    (read_step(std::integral_constant<int, 0>{}, std::integral_constant<int, Q>{}, std::integral_constant<int, Q>{}), ...);
  }(std::make_integer_sequence<int, PD>{});
  __builtin_amdgcn_sched_barrier(0);
  int kt = 0;
  for (; kt + NSTAGE < nk; kt += NSTAGE) round(kt, std::true_type{});
  for (; kt < nk; kt += NSTAGE) round(kt, std::false_type{});

  if (p.a_rowsum != nullptr && tile_n == 0 && wn == 0) {
    T* dst = reinterpret_cast<T*>(p.a_rowsum) + grp * p.rowsum_sg;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const float v = rsum[i] + __shfl_xor(rsum[i], 32, 64);
      const int row = m0 + wm * WM + i * 32 + li;
      if (g == 0 && row < p.m) dst[row] = from_f32<T>((p.flags & RTP_GEMM_ROWSUM_ACCUM) ? to_f32(dst[row]) + v : v);
    }
  }

  // Epilogue in MT passes: pass i stages rows i*32 .. i*32+31 of both tile halves (64 rows of 256 columns, fp32)
  // in the slab memory; every thread then finishes chunks of 8 columns as in the other kernel.
  constexpr int CP = BN + 4;
  float* ct = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    __syncthreads();  // the fragments (first pass) or the previous pass's rows have been read
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        ct[(wm * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * CP + wn * WN + j * 32 + li] = acc[i][j][r];
    __syncthreads();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int mrow = m0 + h * WM + i * 32;
      if (mrow >= p.m) continue;
      finish_tile<T, 32, BN, 512>(p, ct + h * 32 * CP, mrow, n0, tid, grp, zo, zi);
    }
  }
  if (p.trace != nullptr && tid == 0) atomicMax(p.trace + 1, (unsigned long long)wall_clock64());
}

template <typename T, int NSTAGE, int SB, int PD>
static int launch_dma8(hipStream_t s, const GemmArgs& a, bool akc, bool bkc, dim3 grid) {
  const dim3 block(512);
  if (akc && bkc)
    hipLaunchKernelGGL((gemm_dma8_kernel<T, true, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else if (akc && !bkc)
    hipLaunchKernelGGL((gemm_dma8_kernel<T, true, false, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else if (!akc && bkc)
    hipLaunchKernelGGL((gemm_dma8_kernel<T, false, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((gemm_dma8_kernel<T, false, false, NSTAGE, SB, PD>), grid, block, 0, s, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

template <typename T, int BM, int BN, int NSTAGE, int SB, int PD>
static int launch_dma(hipStream_t s, const GemmArgs& a, bool akc, bool bkc, dim3 grid) {
  const dim3 block(512);
  // A row-contiguous operand is staged as k lines of R elements, and a 1 KiB load must cover whole lines (or a
  // whole fraction of one): tile extents that are not powers of two only exist for K-contiguous operands.
  constexpr bool A_RC_OK = (BM & (BM - 1)) == 0, B_RC_OK = (BN & (BN - 1)) == 0;
  if constexpr (!A_RC_OK || !B_RC_OK) {
    RTP_REQUIRE((akc || A_RC_OK) && (bkc || B_RC_OK), "gemm: tile %d x %d needs K-contiguous operands", BM, BN);
    if constexpr (!B_RC_OK && A_RC_OK) {
      if (akc)
        hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, true, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
      else
        hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, false, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
    }
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  } else if (akc && bkc)
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, true, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else if (akc && !bkc)
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, true, false, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else if (!akc && bkc)
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, false, true, NSTAGE, SB, PD>), grid, block, 0, s, a);
  else
    hipLaunchKernelGGL((gemm_dma_kernel<T, BM, BN, false, false, NSTAGE, SB, PD>), grid, block, 0, s, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

// ---------------------------------------------------------------------------------------------
// Tiny batched problems (one attention head at sequence length <= 64: 32 x 32 x 64 per (batch, head)):
// one wavefront per 32 x 32 output block, operands read straight from global memory into MFMA
// fragments (no LDS, no barriers).  Thousands of independent wavefronts hide the load latency.
template <typename T, bool AKC, bool BKC>
__global__ __launch_bounds__(kThreads) void gemm_tiny_kernel(GemmArgs p, long nblocks) {
  constexpr int VEC = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const long blk = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (blk >= nblocks) return;
  const int li = lane & 31, g = lane >> 5;
  const int tiles = p.tiles_m * p.tiles_n;
  const long z = blk / tiles;
  const int tile = (int)(blk % tiles);
  const int m0 = (tile / p.tiles_n) * 32, n0 = (tile % p.tiles_n) * 32;
  const int grp = (int)(z / p.batch), zb = (int)(z % p.batch);
  const long zo = zb / p.zdiv, zi = zb % p.zdiv;
  const T* A = reinterpret_cast<const T*>(p.a) + grp * p.a_sg + zo * p.a_so + zi * p.a_si;
  const T* B = reinterpret_cast<const T*>(p.b) + grp * p.b_sg + zo * p.b_so + zi * p.b_si;

  f32x16 acc[1][1];
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[0][0][r] = 0.0f;

  // fragment of `rows`-row operand X for this lane's row and the VEC k values starting at k
  auto frag = [&](const T* X, long ld, bool kc, bool vec_ok, int row, int rows, int k) {
    union {
      uint4 q;
      T e[VEC];
      Frag<T> f;
    } u;
    if (kc) {
      const T* src = X + (long)row * ld + k;
      if (vec_ok && row < rows && k + VEC <= p.k) {
        u.q = *reinterpret_cast<const uint4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) u.e[e] = (row < rows && k + e < p.k) ? src[e] : (T)0.0f;
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) u.e[e] = (row < rows && k + e < p.k) ? X[(long)(k + e) * ld + row] : (T)0.0f;
    }
    return u.f;
  };

  for (int seg = 0; seg < p.ksegs; ++seg) {
    const T* As = A + seg * p.a_sk;
    const T* Bs = B + seg * p.b_sk;
    for (int k0 = 0; k0 < p.k; k0 += 2 * VEC) {
      const Frag<T> fa = frag(As, p.lda, AKC, p.vec_a, m0 + li, p.m, k0 + g * VEC);
      const Frag<T> fb = frag(Bs, p.ldb, BKC, p.vec_b, n0 + li, p.n, k0 + g * VEC);
      mma(fa, fb, acc[0][0]);
    }
  }
  store_tile<T, 1, 1, 32, 32>(p, acc, m0, n0, 0, 0, li, g, grp, zo, zi);
}

template <typename T, int BM, int BN, int DEPTH, bool FAST>
static int launch_layout(hipStream_t s, const GemmArgs& a, bool akc, bool bkc, dim3 grid) {
  if (akc && bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, true, true, DEPTH, FAST>), grid, dim3(kThreads), 0, s, a);
  else if (akc && !bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, true, false, DEPTH, FAST>), grid, dim3(kThreads), 0, s, a);
  else if (!akc && bkc)
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, false, true, DEPTH, FAST>), grid, dim3(kThreads), 0, s, a);
  else
    hipLaunchKernelGGL((gemm_kernel<T, BM, BN, false, false, DEPTH, FAST>), grid, dim3(kThreads), 0, s, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

static bool mult(int64_t v, int64_t q) { return v % q == 0; }

// Tile shapes, largest first; launch_gemm picks one with a cost model (the 10-layer LM's per-layer problems
// are 1024 x 2048 outputs: 128 tiles of 128x128 but exactly 256, one per CU, of 128x64).
struct TileShape {
  int bm, bn;
  const char* tag;
};
static const TileShape kShapes[7] = {{256, 128, "256x128"}, {128, 128, "128x128"}, {128, 64, "128x64"}, {64, 64, "64x64"},
                                     {128, 192, "128x192"}, {256, 256, "256x256"}, {128, 160, "128x160"}};
constexpr int kNumShapes = 7;

// One wavefront per 32 x 32 block is the better kernel for one attention head at sequence length <= 64.
static bool is_tiny(const rtp_gemm_desc* d) { return d->m <= 64 && d->n <= 64 && d->k * d->ksegs <= 256; }

// Whether the wave-specialised kernel can run the problem.  Its branch-free loads need whole 16-byte vectors:
// aligned operands and extents that are multiples of VEC along each operand's contiguous axis; and a tile's
// byte offsets from its first vector must fit 32 bits (256 rows or k lines of one leading dimension).
// Anything else goes to the guarded small-tile kernel.
template <typename T>
static bool takes_dma_kernel(const rtp_gemm_desc* d) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec_a = mult((int64_t)(uintptr_t)d->a, 16) && mult(d->lda, VEC) && mult(d->a_so, VEC) &&
                     mult(d->a_si, VEC) && mult(d->a_sg, VEC) && mult(d->a_sk, VEC);
  const bool vec_b = mult((int64_t)(uintptr_t)d->b, 16) && mult(d->ldb, VEC) && mult(d->b_so, VEC) &&
                     mult(d->b_si, VEC) && mult(d->b_sg, VEC) && mult(d->b_sk, VEC);
  const bool akc = d->a_kcontig, bkc = d->b_kcontig;
  const int64_t ld_max = ((int64_t)1 << 24) / (int64_t)sizeof(T) - 64;
  return vec_a && vec_b && ((akc || bkc) ? mult(d->k, VEC) : true) && (akc || mult(d->m, VEC)) &&
         (bkc || mult(d->n, VEC)) && d->k > 0 && d->lda <= ld_max && d->ldb <= ld_max;
}

// The fused clip + SGD lives in the epilogue of the wave-specialised kernel; the gradient keeps the compute dtype.
template <typename T>
static bool sgd_fused(const rtp_gemm_desc* d) {
  return !is_tiny(d) && takes_dma_kernel<T>(d) && !(d->flags & (RTP_GEMM_OUT_F32 | RTP_GEMM_RELU)) && !d->c_in &&
         !d->bias && !d->gate;
}

template <typename T>
static bool rowsum_fused(const rtp_gemm_desc* d) {
  return !d->a_kcontig && d->batch == 1 && !is_tiny(d) && takes_dma_kernel<T>(d);
}

// rtp_gemm_warm_next: bytes the next product launched by this host thread requests at its start
static thread_local const void* t_warm_src = nullptr;
static thread_local size_t t_warm_bytes = 0;

template <typename T>
static int launch_gemm(hipStream_t s, const rtp_gemm_desc* d) {
  // the hint of rtp_gemm_warm_next rides in this launch or ends with it
  const void* warm_src = t_warm_src;
  t_warm_src = nullptr;
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
  a.ksegs = (int)d->ksegs;
  a.lda = d->lda;
  a.ldb = d->ldb;
  a.ldc = d->ldc;
  a.ld_cin = d->ld_cin;
  a.ld_gate = d->ld_gate;
  a.batch = (int)d->batch;
  a.zdiv = (int)d->zdiv;
  a.a_so = d->a_so, a.a_si = d->a_si, a.b_so = d->b_so, a.b_si = d->b_si;
  a.c_so = d->c_so, a.c_si = d->c_si, a.cin_so = d->cin_so, a.cin_si = d->cin_si;
  a.gate_so = d->gate_so, a.gate_si = d->gate_si, a.bias_so = d->bias_so, a.bias_si = d->bias_si;
  a.a_sg = d->a_sg, a.b_sg = d->b_sg, a.c_sg = d->c_sg, a.cin_sg = d->cin_sg;
  a.gate_sg = d->gate_sg, a.bias_sg = d->bias_sg;
  a.a_sk = d->a_sk, a.b_sk = d->b_sk, a.bias_sk = d->bias_sk;
  a.alpha = d->alpha;
  a.flags = d->flags;
  a.vec_a = mult((int64_t)(uintptr_t)d->a, 16) && mult(d->lda, VEC) && mult(d->a_so, VEC) && mult(d->a_si, VEC) &&
            mult(d->a_sg, VEC) && mult(d->a_sk, VEC);
  a.vec_b = mult((int64_t)(uintptr_t)d->b, 16) && mult(d->ldb, VEC) && mult(d->b_so, VEC) && mult(d->b_si, VEC) &&
            mult(d->b_sg, VEC) && mult(d->b_sk, VEC);

  {
    auto ok = [](const void* ptr, int64_t ld, int64_t so, int64_t si, int64_t sg) {
      return mult((int64_t)(uintptr_t)ptr, 16) && mult(ld, 8) && mult(so, 8) && mult(si, 8) && mult(sg, 8);
    };
    a.vec_c = mult(d->n, 8) && ok(d->c_out, d->ldc, d->c_so, d->c_si, d->c_sg) &&
              (!d->c_in || ok(d->c_in, d->ld_cin, d->cin_so, d->cin_si, d->cin_sg)) &&
              (!d->gate || ok(d->gate, d->ld_gate, d->gate_so, d->gate_si, d->gate_sg)) &&
              (!d->bias || (ok(d->bias, 8, d->bias_so, d->bias_si, d->bias_sg) && mult(d->bias_sk, 8)));
  }

  const bool akc = d->a_kcontig, bkc = d->b_kcontig;
  const bool fast = takes_dma_kernel<T>(d);
  const int64_t nz = d->batch * d->groups;
  a.a_rowsum = (char*)d->a_rowsum;
  a.rowsum_sg = d->rowsum_sg;
  a.trace = nullptr;
  a.xent_mode = d->xent_mode;
  a.xent_blocks = (int)(d->groups * d->n / 64);
  a.xent_target = (const long*)d->xent_target;
  a.xent_ignore = (long)d->xent_ignore;
  a.xent_part = (float2*)d->xent_part;
  a.xent_tlogit = d->xent_tlogit;
  a.xent_stats = (const float2*)d->xent_stats;
  a.xent_dloss = d->xent_dloss;
  a.xent_scale = d->xent_scale;
  if (d->xent_mode) {
    RTP_REQUIRE(d->xent_mode == 1 || d->xent_mode == 2, "rtp_gemm: xent_mode is 0, 1 or 2");
    RTP_REQUIRE(takes_dma_kernel<T>(d) && !is_tiny(d) && a.vec_c && d->n % 64 == 0 && d->batch == 1 && d->ksegs >= 1 &&
                    d->c_sg == d->n && !(d->flags & (RTP_GEMM_OUT_F32 | RTP_GEMM_RELU)) && !d->c_in && !d->gate,
                "rtp_gemm: the cross-entropy epilogues need vector-aligned operands, groups of a multiple of 64 columns "
                "laid side by side (c_sg == n), an output in the compute dtype and no c_in / ReLU / mask");
    RTP_REQUIRE(d->xent_target && (d->xent_mode == 1 ? (d->xent_part && d->xent_tlogit) : (d->xent_stats && d->xent_dloss)),
                "rtp_gemm: missing cross-entropy operands for mode %d", d->xent_mode);
    RTP_REQUIRE((uintptr_t)d->xent_part % 8 == 0 && (uintptr_t)d->xent_stats % 8 == 0, "rtp_gemm: 8-byte aligned statistics");
  }
  a.sgd_master = (float*)d->sgd_master;
  a.sgd_w = (char*)d->sgd_weights;
  a.sgd_lr = d->sgd_lr;
  a.sgd_clip = d->sgd_clip;
  RTP_REQUIRE(!d->sgd_master || sgd_fused<T>(d),
              "rtp_gemm: sgd_master needs vector-aligned operands, an output in the compute dtype and no c_in / bias / "
              "ReLU / mask (rtp_gemm_sgd_fused)");
  RTP_REQUIRE(d->sgd_master || (!d->sgd_weights && !(d->flags & RTP_GEMM_SGD_SKIP_OUT)),
              "rtp_gemm: sgd_weights / RTP_GEMM_SGD_SKIP_OUT without sgd_master");
  if (d->sgd_master)  // the update's 16-byte accesses: 8 fp32 columns are two of them
    a.vec_c = a.vec_c && mult((int64_t)(uintptr_t)d->sgd_master, 16) &&
              (!d->sgd_weights || mult((int64_t)(uintptr_t)d->sgd_weights, 16));
  RTP_REQUIRE(!d->a_rowsum || rowsum_fused<T>(d),
              "rtp_gemm: a_rowsum needs A stored K x M, batch == 1 and vector-aligned operands (rtp_gemm_rowsum_fused)");
  if (is_tiny(d)) {
    // one wavefront per 32 x 32 block
    a.tiles_m = (int)ceil_div(d->m, 32);
    a.tiles_n = (int)ceil_div(d->n, 32);
    const int64_t nblocks = (int64_t)a.tiles_m * a.tiles_n * nz;
    RTP_REQUIRE(ceil_div(nblocks, 4) < (1ll << 31), "gemm grid too large");
    static const char* const tiny_names[2][2][2] = {
        {{"gemm_f32_tiny_rc_rc", "gemm_f32_tiny_rc_kc"}, {"gemm_f32_tiny_kc_rc", "gemm_f32_tiny_kc_kc"}},
        {{"gemm_bf16_tiny_rc_rc", "gemm_bf16_tiny_rc_kc"}, {"gemm_bf16_tiny_kc_rc", "gemm_bf16_tiny_kc_kc"}}};
    const double mn_ = (double)d->m * (double)d->n * (double)nz, kk_ = (double)d->k * (double)d->ksegs;
    ProfileScope prof(s, tiny_names[sizeof(T) == 2][akc][bkc], 2.0 * mn_ * kk_,
                      ((double)d->m + (double)d->n) * kk_ * nz * sizeof(T) + mn_ * sizeof(T));
    dim3 tgrid((unsigned)ceil_div(nblocks, 4));
    if (akc && bkc)
      hipLaunchKernelGGL((gemm_tiny_kernel<T, true, true>), tgrid, dim3(kThreads), 0, s, a, (long)nblocks);
    else if (akc && !bkc)
      hipLaunchKernelGGL((gemm_tiny_kernel<T, true, false>), tgrid, dim3(kThreads), 0, s, a, (long)nblocks);
    else if (!akc && bkc)
      hipLaunchKernelGGL((gemm_tiny_kernel<T, false, true>), tgrid, dim3(kThreads), 0, s, a, (long)nblocks);
    else
      hipLaunchKernelGGL((gemm_tiny_kernel<T, false, false>), tgrid, dim3(kThreads), 0, s, a, (long)nblocks);
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  }
  // Tile choice by a cost model: the launch runs in ceil(tiles / 256 CUs) rounds, a round costs the tile's
  // measured time per K slab (ns, 4096^3 bf16 on MI355X: bigger tiles do ~30 % more outputs per ns, so what
  // decides is mostly how evenly the tile count fills the CUs) plus a fixed prologue / epilogue.
  static const int forced = [] {
    const char* e = getenv("RTP_GEMM_TILE");  // debugging aid: index into kShapes
    return e ? atoi(e) : -1;
  }();
  static const double slab_ns[kNumShapes] = {966.0, 470.0, 283.0, 167.0, 800.0, 1680.0, 545.0};
  static const int slab_bytes[kNumShapes] = {128, 128, 128, 128, 128, 128, 128};
  int shape = 3;  // 64 x 64 unless the model finds something cheaper
  double best = 0.0;
  for (int i = 0; fast && i < kNumShapes; ++i) {
    // the 256 x 256 kernel is built for 16-bit operands and the plain epilogue, and pays on products that give
    // every CU at least one such tile and contract over 1024 or more (measured against the next best shape:
    // +10 - 25 % at 8192^3, +10 % at 4096^3, +5 - 10 % at K = 1024 .. 1536 when the tiles fill the CUs evenly,
    // -10 % on the MoE layer's time; a loss where it leaves CUs without a tile or K is shorter)
    // (its epilogue is the plain one: the update and the statistics epilogue are never routed to it, forced or not)
    if (i == 5 && (sizeof(T) != 2 || d->sgd_master || d->xent_mode == 1)) continue;
    if (i == 6 && d->xent_mode == 1) continue;  // 160 columns are no whole number of 64-column statistics blocks
    // 128 x 160 is priced at the rate measured where it is meant for -- products of at most two rounds of tiles, such
    // as the LM's logits layer (shards of 1280 columns); larger products keep the shapes measured on large products
    if (i == 6 && ceil_div(d->m, 128) * ceil_div(d->n, 160) * nz > 512 && i != forced) continue;
    if (i == 5 && (ceil_div(d->m, 256) * ceil_div(d->n, 256) * nz < 256 || d->k * d->ksegs < 1024) && i != forced)
      continue;
    // never a tile that is mostly padding: a 32 x 32 problem (one attention head at seq 32) stays at 64 x 64
    if ((!akc && (kShapes[i].bm & (kShapes[i].bm - 1))) || (!bkc && (kShapes[i].bn & (kShapes[i].bn - 1)))) continue;
    if (kShapes[i].bm > 64 && kShapes[i].bm > ceil_div(d->m, 64) * 64) continue;
    if (kShapes[i].bn > 64 && kShapes[i].bn > ceil_div(d->n, 64) * 64) continue;
    const int64_t tiles = ceil_div(d->m, kShapes[i].bm) * ceil_div(d->n, kShapes[i].bn) * nz;
    const double nslabs = (double)ceil_div(d->k * (int64_t)sizeof(T), slab_bytes[i]) * (double)d->ksegs;
    const double cost = (double)ceil_div(tiles, 256) * (nslabs * slab_ns[i] + 3000.0);
    if (best == 0.0 || cost < best || i == forced) {
      best = i == forced ? -1.0 : cost;
      shape = i;
    }
  }
  const TileShape& ts = kShapes[shape];
  a.tiles_m = (int)ceil_div(d->m, ts.bm);
  a.tiles_n = (int)ceil_div(d->n, ts.bn);
  const int64_t nb = (int64_t)a.tiles_m * a.tiles_n;
  RTP_REQUIRE(nb < (1ll << 31) && nz < 65536, "gemm grid too large (%lld tiles, %lld batch*groups)", (long long)nb,
              (long long)nz);
  dim3 grid((unsigned)nb, (unsigned)nz, 1);
  // XCD bricks: among the splits xg*xm*xn == 8 that divide the launch evenly, take the one with the fewest
  // operand bytes per XCD (A rows x K of the brick's row tiles, B likewise; an operand that differs per
  // batch/group entry counts once per entry of the brick).
  a.xg = a.xm = a.xn = 0;
  if (fast) {
    const bool a_per_z = d->batch > 1 || (d->groups > 1 && d->a_sg != 0);
    const bool b_per_z = d->batch > 1 || (d->groups > 1 && d->b_sg != 0);
    double best = 0.0;
    for (int xg = 1; xg <= 8; xg *= 2)
      for (int xm = 1; xg * xm <= 8; xm *= 2) {
        const int xn = 8 / (xg * xm);
        if (nz % xg || a.tiles_m % xm || a.tiles_n % xn) continue;
        const double zb = (double)(nz / xg);
        const double cost = (double)(a.tiles_m / xm) * ts.bm * (a_per_z ? zb : 1.0) +
                            (double)(a.tiles_n / xn) * ts.bn * (b_per_z ? zb : 1.0);
        if (a.xg == 0 || cost < best) {
          best = cost;
          a.xg = xg;
          a.xm = xm;
          a.xn = xn;
        }
      }
  }

  a.d_batch = make_fastdiv((unsigned)d->batch);
  a.d_zdiv = make_fastdiv((unsigned)d->zdiv);
  a.d_tiles_n = make_fastdiv((unsigned)a.tiles_n);
  {
    const int nbk = a.xg ? a.tiles_n / a.xn : 1, mbk = a.xg ? a.tiles_m / a.xm : 1;
    // Panel = prow x pcol tiles, about one round of an XCD's 32 CUs.  pcol: the widest divisor of nbk (at most 32)
    // whose strip of B tiles (pcol * BN rows x all of K) stays within ~3 MB of the XCD's 4 MB L2 -- the A rows stream
    // past the strip once, so the L2 fills are about A * nbk / pcol + B per brick.  prow: the tallest divisor of mbk
    // that keeps the panel within 32 tiles.
    const double b_tile_bytes = (double)ts.bn * (double)d->k * (double)d->ksegs * sizeof(T);
    int pcol = 1;
    for (int c = 2; c <= 32 && c <= nbk; ++c)
      if (nbk % c == 0 && c * b_tile_bytes <= 3.0 * 1024 * 1024) pcol = c;
    // A contraction so long that not even two B tiles fit: nothing stays in the L2 from one panel to the next, and
    // what counts is the block of tiles that run at the same time and walk K side by side -- as square as it gets
    // (a 16 x 1 column shares one B tile but streams 16 A tiles; 8 x 4 streams 12 tile-operands for 32 CUs).
    if (pcol == 1)
      for (int c = 2; c <= 4 && c <= nbk; ++c)
        if (nbk % c == 0) pcol = c;
    int prow = 1;
    for (int r = 2; r * pcol <= 32 && r <= mbk; ++r)
      if (mbk % r == 0) prow = r;
    a.mbk = mbk, a.nbk = nbk;
    a.prow = prow, a.pcol = pcol;
    a.d_brick = make_fastdiv((unsigned)(nbk * mbk));
    a.d_panel = make_fastdiv((unsigned)(prow * pcol));
    a.d_prow = make_fastdiv((unsigned)prow);
    a.d_pm = make_fastdiv((unsigned)(mbk / prow));
  }
  a.xn_shift = a.xn == 8 ? 3 : a.xn == 4 ? 2 : a.xn == 2 ? 1 : 0;
  a.xm_shift = a.xm == 8 ? 3 : a.xm == 4 ? 2 : a.xm == 2 ? 1 : 0;
  a.zbk = a.xg ? (int)(nz / a.xg) : 0;

  // variant name = the kernel template instance, e.g. gemm_bf16_128x64_kc_kc
  static const char* const layout_tag[2][2] = {{"rc_rc", "rc_kc"}, {"kc_rc", "kc_kc"}};
  static thread_local char names[2][kNumShapes + 1][2][2][40];
  char* name = names[sizeof(T) == 2][fast ? shape : kNumShapes][akc][bkc];
  if (!name[0])
    snprintf(name, 40, "gemm_%s_%s_%s", sizeof(T) == 2 ? "bf16" : "f32", fast ? ts.tag : "64x64_guarded",
             layout_tag[akc][bkc]);
  const double mn = (double)d->m * (double)d->n * (double)nz;
  const double kk = (double)d->k * (double)d->ksegs;
  const double out_sz = (d->flags & RTP_GEMM_OUT_F32) ? 4.0 : (double)sizeof(T);
  const double cin_sz = d->c_in ? ((d->flags & RTP_GEMM_CIN_F32) ? 4.0 : (double)sizeof(T)) : 0.0;
  // operands once + the output (and addend); a fused update reads and writes the fp32 parameters and writes their copy
  const double upd_sz = d->sgd_master ? 8.0 + (d->sgd_weights ? (double)sizeof(T) : 0.0) -
                                            ((d->flags & RTP_GEMM_SGD_SKIP_OUT) ? out_sz : 0.0)
                                      : 0.0;
  // An operand that every group / batch entry / K segment reads from the same address (stride 0: the activations of a
  // column layer's forward and weight-gradient products) is counted once, not once per shard.
  const auto copies = [&](int64_t so, int64_t si, int64_t sg, int64_t sk) {
    const double per_batch = (d->batch > 1 && (so != 0 || si != 0)) ? (double)d->batch : 1.0;
    const double per_group = (d->groups > 1 && sg != 0) ? (double)d->groups : 1.0;
    const double per_kseg = (d->ksegs > 1 && sk != 0) ? (double)d->ksegs : 1.0;
    return per_batch * per_group * per_kseg;
  };
  const double bytes = ((double)d->m * copies(d->a_so, d->a_si, d->a_sg, d->a_sk) +
                        (double)d->n * copies(d->b_so, d->b_si, d->b_sg, d->b_sk)) * (double)d->k * sizeof(T) +
                       mn * (out_sz + cin_sz + upd_sz);
  ProfileScope prof(s, name, 2.0 * mn * kk, bytes);
  a.trace = fast ? prof.trace_slot() : nullptr;
  a.warm = nullptr;
  a.warm_bytes = 0;
  if (!fast) return launch_layout<T, 64, 64, 1, false>(s, a, akc, bkc, grid);
  if (shape != 5 && warm_src != nullptr) {
    a.warm = (const char*)warm_src;
    a.warm_bytes = (long)t_warm_bytes;
  }
  switch (shape) {
    case 0:
      return launch_dma<T, 256, 128, 3, 128, 1>(s, a, akc, bkc, grid);
    case 1:
      // prefetch distance 1: as fast as 3 on every measured shape, and 168 instead of 213 registers per wave for
      // the weight-gradient layout -- with two such waves per SIMD the 120-register waves of the LayerNorm backward
      // kernel on the other stream fit beside them instead of waiting for a workgroup to leave the CU
      return launch_dma<T, 128, 128, 4, 128, 1>(s, a, akc, bkc, grid);
    case 2:
      return launch_dma<T, 128, 64, 5, 128, 4>(s, a, akc, bkc, grid);
    case 4:
      return launch_dma<T, 128, 192, 3, 128, 2>(s, a, akc, bkc, grid);
    case 6:
      // 4 x 1 wave tiles of 32 x 160: a layer whose shards are 1280 columns wide (the LM's logits) is 8 tiles per
      // shard and fills the CUs in two even rounds where 128 x 128 tiles need two and a half
      return launch_dma<T, 128, 160, 4, 128, 1>(s, a, akc, bkc, grid);
    case 5:
      if constexpr (sizeof(T) == 2) return launch_dma8<T, 2, 128, 1>(s, a, akc, bkc, grid);
      return fail(RTP_ERR_ARG, "gemm: no 256 x 256 kernel for this dtype");
    default:
      return launch_dma<T, 64, 64, 4, 128, 3>(s, a, akc, bkc, grid);
  }
}

// ---------------------------------------------------------------------------------------------
// Column sums (bias gradients) in two deterministic passes: 64 columns x a block of rows per
// workgroup into fp32 partials, then a fixed-order sum of the partials.
constexpr int kColsumRows = 64;

template <typename T>
__global__ __launch_bounds__(kThreads) void colsum_partial_kernel(const T* x, long m, long n, long ld, float* part) {
  __shared__ float red[4][64];
  const int c = threadIdx.x & 63, ph = threadIdx.x >> 6;
  const long col = (long)blockIdx.x * 64 + c;
  const long r0 = (long)blockIdx.y * kColsumRows;
  const long r1 = r0 + kColsumRows < m ? r0 + kColsumRows : m;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < n) {
    long r = r0 + ph;
    for (; r + 12 < r1; r += 16) {
      s0 += to_f32(x[r * ld + col]);
      s1 += to_f32(x[(r + 4) * ld + col]);
      s2 += to_f32(x[(r + 8) * ld + col]);
      s3 += to_f32(x[(r + 12) * ld + col]);
    }
    for (; r < r1; r += 4) s0 += to_f32(x[r * ld + col]);
  }
  red[ph][c] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (ph == 0 && col < n) part[(long)blockIdx.y * n + col] = (red[0][c] + red[1][c]) + (red[2][c] + red[3][c]);
}

// Single-pass variant for a few thousand rows: one workgroup of 512 threads owns 32 columns; each thread walks
// its rows with 16-byte loads (VEC columns, 4 loads in flight), and the per-thread sums are combined through LDS
// in a fixed order (row groups in 4 quarters, then the quarters).
constexpr int kOnepassThreads = 512, kOnepassCols = 32;
template <typename T>
__global__ __launch_bounds__(kOnepassThreads) void colsum_onepass_kernel(const T* x, long m, long n, long ld, void* out,
                                                                         long seg, long seg_stride, int out_f32,
                                                                         int accumulate) {
  constexpr int VEC = 16 / sizeof(T), LPR = kOnepassCols / VEC, RG = kOnepassThreads / LPR;
  __shared__ float red[RG][kOnepassCols + 1];
  __shared__ float quarter[4][kOnepassCols];
  const int cl = (threadIdx.x % LPR) * VEC, rg = threadIdx.x / LPR;
  const long col = (long)blockIdx.x * kOnepassCols + cl;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
  if (col < n) {  // n is a multiple of VEC, so the vector is wholly inside
    union V {
      uint4 q;
      T e[VEC];
    };
    const T* src = x + col;
    long r = rg;
    for (; r + 3 * RG < m; r += 4 * RG) {
      V u0, u1, u2, u3;
      u0.q = *reinterpret_cast<const uint4*>(src + r * ld);
      u1.q = *reinterpret_cast<const uint4*>(src + (r + RG) * ld);
      u2.q = *reinterpret_cast<const uint4*>(src + (r + 2 * RG) * ld);
      u3.q = *reinterpret_cast<const uint4*>(src + (r + 3 * RG) * ld);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += (to_f32(u0.e[e]) + to_f32(u1.e[e])) + (to_f32(u2.e[e]) + to_f32(u3.e[e]));
    }
    for (; r < m; r += RG) {
      V u;
      u.q = *reinterpret_cast<const uint4*>(src + r * ld);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += to_f32(u.e[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) red[rg][cl + e] = acc[e];
  __syncthreads();
  if (threadIdx.x < 4 * kOnepassCols) {
    const int c = threadIdx.x % kOnepassCols, qd = threadIdx.x / kOnepassCols;
    float v = 0.0f;
    for (int r = qd * (RG / 4); r < (qd + 1) * (RG / 4); ++r) v += red[r][c];
    quarter[qd][c] = v;
  }
  __syncthreads();
  const long c = (long)blockIdx.x * kOnepassCols + threadIdx.x;
  if (threadIdx.x < kOnepassCols && c < n) {
    const int t = threadIdx.x;
    const float v = (quarter[0][t] + quarter[1][t]) + (quarter[2][t] + quarter[3][t]);
    const long o = (c / seg) * seg_stride + c % seg;
    if (out_f32) {
      float* dst = reinterpret_cast<float*>(out);
      dst[o] = accumulate ? dst[o] + v : v;
    } else {
      T* dst = reinterpret_cast<T*>(out);
      dst[o] = from_f32<T>(accumulate ? to_f32(dst[o]) + v : v);
    }
  }
}

// out index of column c: (c / seg) * seg_stride + c % seg  (bias slices of consecutive shards sit
// seg_stride elements apart in the flat gradient buffer).
template <typename T>
__global__ __launch_bounds__(kThreads) void colsum_final_kernel(const float* part, long nparts, long n, void* out,
                                                                long seg, long seg_stride, int out_f32,
                                                                int accumulate) {
  const long col = (long)blockIdx.x * kThreads + threadIdx.x;
  if (col >= n) return;
  float v = 0.0f;
  for (long p = 0; p < nparts; ++p) v += part[p * n + col];
  const long o = (col / seg) * seg_stride + col % seg;
  if (out_f32) {
    float* dst = reinterpret_cast<float*>(out);
    dst[o] = accumulate ? dst[o] + v : v;
  } else {
    T* dst = reinterpret_cast<T*>(out);
    dst[o] = from_f32<T>(accumulate ? to_f32(dst[o]) + v : v);
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
  RTP_REQUIRE(d->batch >= 1 && d->zdiv >= 1 && d->groups >= 1 && d->ksegs >= 1,
              "rtp_gemm: batch=%lld zdiv=%lld groups=%lld ksegs=%lld must be >= 1", (long long)d->batch,
              (long long)d->zdiv, (long long)d->groups, (long long)d->ksegs);
  RTP_REQUIRE(d->k * d->ksegs < (1ll << 31), "rtp_gemm: total contraction length exceeds int32");
  RTP_REQUIRE(d->lda >= 1 && d->ldb >= 1 && d->ldc >= 1, "rtp_gemm: leading dimensions must be >= 1");
  RTP_REQUIRE(!d->c_in || d->ld_cin >= 1, "rtp_gemm: ld_cin must be >= 1 when c_in is given");
  RTP_REQUIRE(!d->gate || d->ld_gate >= 1, "rtp_gemm: ld_gate must be >= 1 when gate is given");
  if (d->m == 0 || d->n == 0) return RTP_OK;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == RTP_F32) return launch_gemm<float>(s, d);
  if (dtype == RTP_BF16) return launch_gemm<bf16_t>(s, d);
  return fail(RTP_ERR_ARG, "rtp_gemm: unknown dtype %d", dtype);
}

extern "C" int rtp_gemm_rowsum_fused(int dtype, const rtp_gemm_desc* d) {
  using namespace rtp;
  if (!d || !d->a || !d->b || d->m <= 0 || d->n <= 0 || d->k <= 0 || d->groups < 1 || d->ksegs < 1) return 0;
  if (dtype == RTP_F32) return rowsum_fused<float>(d) ? 1 : 0;
  if (dtype == RTP_BF16) return rowsum_fused<bf16_t>(d) ? 1 : 0;
  return 0;
}

extern "C" int rtp_gemm_warm_next(const void* src, size_t bytes) {
  RTP_REQUIRE(((uintptr_t)src & 15) == 0, "rtp_gemm_warm_next: source must be 16-byte aligned");
  rtp::t_warm_src = bytes ? src : nullptr;
  rtp::t_warm_bytes = bytes;
  return RTP_OK;
}

extern "C" int rtp_gemm_sgd_fused(int dtype, const rtp_gemm_desc* d) {
  using namespace rtp;
  if (!d || !d->a || !d->b || d->m <= 0 || d->n <= 0 || d->k <= 0 || d->groups < 1 || d->ksegs < 1) return 0;
  if (dtype == RTP_F32) return sgd_fused<float>(d) ? 1 : 0;
  if (dtype == RTP_BF16) return sgd_fused<bf16_t>(d) ? 1 : 0;
  return 0;
}

extern "C" size_t rtp_gemm_desc_size(void) { return sizeof(rtp_gemm_desc); }

extern "C" size_t rtp_colsum_workspace_bytes(int64_t m, int64_t n) {
  using namespace rtp;
  if (m <= 0 || n <= 0) return 256;
  return (size_t)(ceil_div(m, kColsumRows) * n * 4 + 256);
}

extern "C" int rtp_colsum(void* stream, int dtype, const void* x, int64_t m, int64_t n, int64_t ld, void* out,
                          int out_f32, int accumulate, int64_t seg, int64_t seg_stride, void* workspace,
                          size_t workspace_bytes) {
  using namespace rtp;
  RTP_REQUIRE(x && out && workspace, "rtp_colsum: null pointer");
  RTP_REQUIRE(m >= 0 && n >= 0 && ld >= n, "rtp_colsum: bad shape m=%lld n=%lld ld=%lld", (long long)m,
              (long long)n, (long long)ld);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_colsum: unknown dtype %d", dtype);
  if (n == 0) return RTP_OK;
  if (seg <= 0) {
    seg = n;
    seg_stride = n;
  }
  RTP_REQUIRE(seg_stride >= seg, "rtp_colsum: seg_stride %lld < seg %lld", (long long)seg_stride, (long long)seg);
  const int64_t nparts = std::max<int64_t>(1, ceil_div(m, kColsumRows));
  RTP_REQUIRE(nparts < 65536, "rtp_colsum: too many rows");
  if (workspace_bytes < (size_t)(nparts * n * 4))
    return fail(RTP_ERR_WORKSPACE, "rtp_colsum: workspace %zu < required %lld", workspace_bytes,
                (long long)(nparts * n * 4));
  hipStream_t s = (hipStream_t)stream;
  float* part = (float*)workspace;
  ProfileScope prof(s, "colsum", (double)m * n, (double)m * n * (dtype == RTP_F32 ? 4 : 2));
  const int vec = dtype == RTP_F32 ? 4 : 8;
  if (m <= 4096 && (uintptr_t)x % 16 == 0 && ld % vec == 0 && n % vec == 0) {
    dim3 g1((unsigned)ceil_div(n, kOnepassCols));
    if (dtype == RTP_F32)
      hipLaunchKernelGGL(colsum_onepass_kernel<float>, g1, dim3(kOnepassThreads), 0, s, (const float*)x, (long)m, (long)n,
                         (long)ld, out, (long)seg, (long)seg_stride, 1, accumulate);
    else
      hipLaunchKernelGGL(colsum_onepass_kernel<bf16_t>, g1, dim3(kOnepassThreads), 0, s, (const bf16_t*)x, (long)m, (long)n,
                         (long)ld, out, (long)seg, (long)seg_stride, out_f32, accumulate);
    RTP_LAUNCH_CHECK();
    return RTP_OK;
  }
  dim3 grid((unsigned)ceil_div(n, 64), (unsigned)nparts);
  dim3 grid2((unsigned)ceil_div(n, kThreads));
  if (dtype == RTP_F32) {
    hipLaunchKernelGGL(colsum_partial_kernel<float>, grid, dim3(kThreads), 0, s, (const float*)x, (long)m, (long)n,
                       (long)ld, part);
    hipLaunchKernelGGL(colsum_final_kernel<float>, grid2, dim3(kThreads), 0, s, part, (long)nparts, (long)n, out,
                       (long)seg, (long)seg_stride, 1, accumulate);
  } else {
    hipLaunchKernelGGL(colsum_partial_kernel<bf16_t>, grid, dim3(kThreads), 0, s, (const bf16_t*)x, (long)m, (long)n,
                       (long)ld, part);
    hipLaunchKernelGGL(colsum_final_kernel<bf16_t>, grid2, dim3(kThreads), 0, s, part, (long)nparts, (long)n, out,
                       (long)seg, (long)seg_stride, out_f32, accumulate);
  }
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
