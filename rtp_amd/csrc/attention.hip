// Fused attention core for short sequences (L <= 32), bf16: one wavefront owns one (group, batch, head)
// problem and keeps scores, probabilities and their gradients in registers.
//
//   forward : S^T = K Q^T (MFMA) -> softmax over keys (fp32, in registers) -> P stored (bf16) -> O^T = V^T P^T (MFMA)
//   backward: dP^T = V dO^T -> dS = scale * P o (dP - rowsum(dP o P)) -> dQ^T = K^T dS^T, dK^T = Q^T dS, dV^T = dO^T P
//
// The transposed products are chosen so that the softmax axis (keys) lies along the accumulator REGISTERS
// of a lane: MFMA 32x32 accumulator register r of lane (li, g) is row 8*(r/4) + 4*g + r%4, column li.  With
// rows = keys and columns = queries a lane holds 16 keys of one query, its partner lane (li, 1-g) the other 16,
// so a row reduction is 15 in-lane operations and one cross-lane exchange.  The same registers, rounded to
// bf16, are directly the B operand of the next product: an MFMA contracts over "k slots" (8 per lane and
// instruction), and which key sits in which slot is free as long as A and B agree; the A operand (V^T, K^T)
// is gathered from LDS in the matching order.
#include "common.h"

namespace rtp {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct AttnArgs {
  // element (l, b, h, g, dd) of q/k/v (and dq/dk/dv) at base + l*s_l + b*s_b + h*s_h + g*s_g + dd
  const bf16_t *q, *k, *v;
  bf16_t *dq, *dk, *dv;
  long s_l, s_b, s_h, s_g;
  // element (l, b, h, g, dd) of o / dout at base + l*o_l + b*o_b + h*o_h + g*o_g + dd
  bf16_t* o;
  const bf16_t* dout;
  long o_l, o_b, o_h, o_g;
  bf16_t* p;          // probabilities [G][N][H][L][L]
  const float* mask;   // additive [L][L] or null
  const float* kbias;  // additive per (batch, key) [N][L] or null (a key padding mask: 0 / -inf)
  int causal;
  float scale;
  int L, N, H;
  long nprob;  // G * N * H
};

constexpr int kSeqMax = 32;
constexpr int kPPitch = kSeqMax + 8;  // row pitch of the P / dS tiles in LDS

// NT tiles of 32 x D (rows beyond L zero) global -> LDS with 16-byte accesses, row pitch D + 8 elements.  Every
// load of every tile is issued before the first LDS write, and without branches (rows beyond L re-read row 0 and are
// zeroed afterwards): a wave owns its problem alone, so a load that waits for the previous one to land puts a full
// trip to memory on the kernel's critical path, and there would be a dozen of them.
template <int D, int NT>
struct TileRegs {
  static constexpr int CPR = D / 8, NIT = kSeqMax * CPR / kWave;
  uint4 val[NT][NIT];
  __device__ __forceinline__ void fetch(const bf16_t* const (&base)[NT], const long (&s_l)[NT], int L, int lane) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + it * kWave, row = c / CPR, cc = c % CPR;
        val[t][it] = *reinterpret_cast<const uint4*>(base[t] + (row < L ? row : 0) * s_l[t] + cc * 8);
      }
  }
  __device__ __forceinline__ void commit(bf16_t* const (&tile)[NT], int L, int lane) const {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + it * kWave, row = c / CPR, cc = c % CPR;
        *reinterpret_cast<uint4*>(tile[t] + row * (D + 8) + cc * 8) = row < L ? val[t][it] : make_uint4(0u, 0u, 0u, 0u);
      }
  }
};

// Operand fragment with the contraction index contiguous in the tile: row li, elements 16*ks + 8*g ...
__device__ __forceinline__ bf16x8 frag_rowmajor(const bf16_t* tile, int pitch, int li, int g, int ks) {
  return *reinterpret_cast<const bf16x8*>(tile + li * pitch + 16 * ks + 8 * g);
}
// Operand fragments whose contraction index is the tile ROW come through the LDS's transposing read: per group of
// 16 lanes it takes a 4 x 16 block (lane t supplies the address of 4 consecutive elements of row t/4 at column
// 4*(t%4)) and hands lane t the 4 elements of column t.  Two of them make the 8 contraction slots of a lane.
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ s16x4 lds_transposed4(const bf16_t* tile, int pitch, int row0, int col0, int t) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + (row0 + (t >> 2)) * pitch + col0 + 4 * (t & 3)));
}
__device__ __forceinline__ bf16x8 join(s16x4 lo, s16x4 hi) {
  union {
    s16x4 h[2];
    bf16x8 f;
  } u;
  u.h[0] = lo, u.h[1] = hi;
  return u.f;
}
// Fragment of the lane that owns tile column col0 + (lane & 31).  ACCUMULATOR order: slot e of instruction m in lane
// group g is row 8*(2m + e/4) + 4g + e%4 (the row that accumulator register 8m + e of that lane group holds).
__device__ __forceinline__ bf16x8 gather_acc_order(const bf16_t* tile, int pitch, int col0, int m, int lane) {
  const int t = lane & 15, c = col0 + (lane & 16), g = lane >> 5;
  return join(lds_transposed4(tile, pitch, 16 * m + 4 * g, c, t), lds_transposed4(tile, pitch, 16 * m + 8 + 4 * g, c, t));
}
// Natural order: slot e of instruction m in lane group g is row 16m + 8g + e.
__device__ __forceinline__ bf16x8 gather_natural(const bf16_t* tile, int pitch, int col0, int m, int lane) {
  const int t = lane & 15, c = col0 + (lane & 16), g = lane >> 5;
  return join(lds_transposed4(tile, pitch, 16 * m + 8 * g, c, t), lds_transposed4(tile, pitch, 16 * m + 8 * g + 4, c, t));
}

// Accumulator (rows = feature dd, columns = sequence position li) -> dst[li][32*db + dd], 4 consecutive dd
// (8 bytes) per store.
__device__ __forceinline__ void store_transposed(bf16_t* dst_row, int db, int g, const f32x16& acc) {
#pragma unroll
  for (int a4 = 0; a4 < 4; ++a4) {
    union {
      uint2 u;
      bf16_t e[4];
    } pk;
#pragma unroll
    for (int e = 0; e < 4; ++e) pk.e[e] = from_f32<bf16_t>(acc[4 * a4 + e]);
    *reinterpret_cast<uint2*>(dst_row + 32 * db + 8 * a4 + 4 * g) = pk.u;
  }
}

struct Problem {
  long z, qkv_off, o_off;
  int b;
  bool live;
};
// The wave index is made scalar and the problem index is split by 32-bit divisions (the host keeps nprob below 2^31):
// 64-bit divisions are software loops of ~140 instructions each, in front of the kernel's first load.
__device__ __forceinline__ Problem locate(const AttnArgs& a, int waves_per_block) {
  Problem pr;
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  unsigned z = blockIdx.x * (unsigned)waves_per_block + wave;
  pr.live = z < (unsigned)a.nprob;
  if (!pr.live) z = (unsigned)a.nprob - 1;  // idle waves redo the last problem and store nothing
  pr.z = z;
  const unsigned zh = z / (unsigned)a.H, h = z - zh * (unsigned)a.H;
  const unsigned g = zh / (unsigned)a.N, b = zh - g * (unsigned)a.N;
  pr.qkv_off = (long)b * a.s_b + (long)h * a.s_h + (long)g * a.s_g;
  pr.o_off = (long)b * a.o_b + (long)h * a.o_h + (long)g * a.o_g;
  pr.b = (int)b;
  return pr;
}

template <int DB, int NWV>
__global__ __launch_bounds__(NWV * 64) void attn_fwd_small_kernel(AttnArgs a) {
  touch_kernel_arguments<sizeof(AttnArgs)>();
  constexpr int D = 32 * DB, P = D + 8;
  __shared__ __attribute__((aligned(16))) bf16_t tiles[NWV][3][kSeqMax * P];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const Problem pr = locate(a, NWV);
  bf16_t* Qs = tiles[wave][0];
  bf16_t* Ks = tiles[wave][1];
  bf16_t* Vs = tiles[wave][2];
  // Tiles first, then the additive mask values of this lane's 16 (query li, key) pairs; the mask is not looked at
  // before the softmax, so its loads are in flight during the tile hand-over and the first product.
  const bool qlive = li < a.L;
  // keys come in runs of 4: with L % 4 == 0 whole runs are inside or outside the sequence (8-byte accesses to P)
  const bool quads = a.L % 4 == 0 && reinterpret_cast<uintptr_t>(a.p) % 8 == 0;
  TileRegs<D, 3> regs;
  {
    const bf16_t* const src[3] = {a.q + pr.qkv_off, a.k + pr.qkv_off, a.v + pr.qkv_off};
    const long sl[3] = {a.s_l, a.s_l, a.s_l};
    regs.fetch(src, sl, a.L, lane);
  }
  float mk[16];
  const bool mask_quads = a.L % 4 == 0 && reinterpret_cast<uintptr_t>(a.mask) % 16 == 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) mk[r] = 0.0f;
  if (a.mask) {
    if (mask_quads) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int key0 = 8 * a4 + 4 * g;
        const float4 m4 = *reinterpret_cast<const float4*>(a.mask + ((qlive && key0 < a.L) ? li * a.L + key0 : 0));
        mk[4 * a4 + 0] = m4.x, mk[4 * a4 + 1] = m4.y, mk[4 * a4 + 2] = m4.z, mk[4 * a4 + 3] = m4.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = 8 * (r >> 2) + 4 * g + (r & 3);
        mk[r] = a.mask[(qlive && key < a.L) ? li * a.L + key : 0];
      }
    }
  }
  float kb[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) kb[r] = 0.0f;
  if (a.kbias) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 8 * (r >> 2) + 4 * g + (r & 3);
      kb[r] = a.kbias[(long)pr.b * a.L + (key < a.L ? key : 0)];
    }
  }
  {
    bf16_t* const tl[3] = {Qs, Ks, Vs};
    regs.commit(tl, a.L, lane);
  }
  __syncthreads();

  // S^T[key][query]
  f32x16 s;
#pragma unroll
  for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Ks, P, li, g, ks), frag_rowmajor(Qs, P, li, g, ks), s, 0,
                                                0, 0);

  // softmax over the keys of query li, in the log2 domain (scale * log2 e in one FMA, the hardware 2^x)
  constexpr float kLog2eSmall = 1.44269504088896340736f;
  const float scale2 = a.scale * kLog2eSmall;
  float val[16];
  float mx = -INFINITY;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int key = 8 * (r >> 2) + 4 * g + (r & 3);
    const bool visible = key < a.L && (!a.causal || key <= li);
    // outside the sequence: unrelated mask entries
    const float x = fmaf(s[r], scale2, ((qlive && key < a.L) ? (mk[r] + kb[r]) * kLog2eSmall : 0.0f));
    val[r] = visible ? x : -INFINITY;
    mx = fmaxf(mx, val[r]);
  }
  mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
  float sum = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    val[r] = __builtin_amdgcn_exp2f(val[r] - mx);  // hidden keys: 2^(-inf) = 0; every key hidden: NaN, as torch gives
    sum += val[r];
  }
  sum += __shfl_xor(sum, 32, kWave);
  const float inv = 1.0f / sum;
  bf16x8 pb[2];
#pragma unroll
  for (int r = 0; r < 16; ++r) pb[r >> 3][r & 7] = from_f32<bf16_t>(val[r] * inv);
  if (pr.live && qlive) {
    bf16_t* prow = a.p + (pr.z * a.L + li) * a.L;
    if (quads) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        union {
          uint2 u;
          bf16_t e[4];
        } pk;
#pragma unroll
        for (int e = 0; e < 4; ++e) pk.e[e] = pb[(4 * a4 + e) >> 3][(4 * a4 + e) & 7];
        if (8 * a4 + 4 * g < a.L) *reinterpret_cast<uint2*>(prow + 8 * a4 + 4 * g) = pk.u;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = 8 * (r >> 2) + 4 * g + (r & 3);
        if (key < a.L) prow[key] = pb[r >> 3][r & 7];
      }
    }
  }

  // O^T[dd][query] = sum_key V[key][dd] P[query][key]
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Vs, P, 32 * db, m, lane), pb[m], acc, 0, 0, 0);
    if (pr.live && qlive) store_transposed(a.o + pr.o_off + li * a.o_l, db, g, acc);
  }
}

template <int DB, int NWV>
__global__ __launch_bounds__(NWV * 64) void attn_bwd_small_kernel(AttnArgs a) {
  touch_kernel_arguments<sizeof(AttnArgs)>();
  constexpr int D = 32 * DB, P = D + 8;
  __shared__ __attribute__((aligned(16))) bf16_t tiles[NWV][4][kSeqMax * P];
  __shared__ __attribute__((aligned(16))) bf16_t ptiles[NWV][2][kSeqMax * kPPitch];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const Problem pr = locate(a, NWV);
  bf16_t* Qs = tiles[wave][0];
  bf16_t* Ks = tiles[wave][1];
  bf16_t* Vs = tiles[wave][2];
  bf16_t* Gs = tiles[wave][3];  // dO
  bf16_t* DSs = ptiles[wave][0];
  bf16_t* Ps = ptiles[wave][1];
  // Tiles first, then this lane's 16 probabilities P[query li][key]: they are not needed before dP is there.
  const bool qlive = li < a.L;
  TileRegs<D, 4> regs;
  {
    const bf16_t* const src[4] = {a.q + pr.qkv_off, a.k + pr.qkv_off, a.v + pr.qkv_off, a.dout + pr.o_off};
    const long sl[4] = {a.s_l, a.s_l, a.s_l, a.o_l};
    regs.fetch(src, sl, a.L, lane);
  }
  const bf16_t* prow = a.p + (pr.z * a.L + (qlive ? li : 0)) * a.L;
  // keys come in runs of 4: with L % 4 == 0 whole runs are inside or outside the sequence (8-byte accesses to P)
  const bool quads = a.L % 4 == 0 && reinterpret_cast<uintptr_t>(a.p) % 8 == 0;
  union {
    uint2 u;
    bf16_t e[4];
  } p4[4];
  bf16_t p1[16];
  if (quads) {
#pragma unroll
    for (int a4 = 0; a4 < 4; ++a4) {
      const int key0 = 8 * a4 + 4 * g;
      p4[a4].u = *reinterpret_cast<const uint2*>(prow + ((qlive && key0 < a.L) ? key0 : 0));
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 8 * (r >> 2) + 4 * g + (r & 3);
      p1[r] = prow[(qlive && key < a.L) ? key : 0];
    }
  }
  {
    bf16_t* const tl[4] = {Qs, Ks, Vs, Gs};
    regs.commit(tl, a.L, lane);
  }
  __syncthreads();

  // dP^T[key][query] = sum_dd V[key][dd] dO[query][dd]
  f32x16 dp;
#pragma unroll
  for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks)
    dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Vs, P, li, g, ks), frag_rowmajor(Gs, P, li, g, ks), dp, 0,
                                                 0, 0);
  float pv[16];
  float dot = 0.0f;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int key = 8 * (r >> 2) + 4 * g + (r & 3);
    const float pr_ = to_f32(quads ? p4[r >> 2].e[r & 3] : p1[r]);
    pv[r] = (qlive && key < a.L) ? pr_ : 0.0f;
    dot += pv[r] * dp[r];
  }
  dot += __shfl_xor(dot, 32, kWave);
  bf16x8 dsb[2];
#pragma unroll
  for (int r = 0; r < 16; ++r) dsb[r >> 3][r & 7] = from_f32<bf16_t>(a.scale * pv[r] * (dp[r] - dot));
  // dS and P as [query][key] tiles for the products that contract over the queries
#pragma unroll
  for (int a4 = 0; a4 < 4; ++a4) {
    union {
      uint2 u;
      bf16_t e[4];
    } d4, p4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      d4.e[e] = dsb[(4 * a4 + e) >> 3][(4 * a4 + e) & 7];
      p4.e[e] = from_f32<bf16_t>(pv[4 * a4 + e]);
    }
    *reinterpret_cast<uint2*>(DSs + li * kPPitch + 8 * a4 + 4 * g) = d4.u;
    *reinterpret_cast<uint2*>(Ps + li * kPPitch + 8 * a4 + 4 * g) = p4.u;
  }
  __syncthreads();

  const bool store = pr.live && qlive;  // li is the query for dQ and the key for dK / dV; both run to L
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    f32x16 acc;
    // dQ^T[dd][query] = sum_key K[key][dd] dS[query][key]
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Ks, P, 32 * db, m, lane), dsb[m], acc, 0, 0, 0);
    if (store) store_transposed(a.dq + pr.qkv_off + li * a.s_l, db, g, acc);
    // dK^T[dd][key] = sum_query Q[query][dd] dS[query][key]
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_natural(Qs, P, 32 * db, m, lane),
                                                    gather_natural(DSs, kPPitch, 0, m, lane), acc, 0, 0, 0);
    if (store) store_transposed(a.dk + pr.qkv_off + li * a.s_l, db, g, acc);
    // dV^T[dd][key] = sum_query dO[query][dd] P[query][key]
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
    for (int m = 0; m < 2; ++m)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_natural(Gs, P, 32 * db, m, lane),
                                                    gather_natural(Ps, kPPitch, 0, m, lane), acc, 0, 0, 0);
    if (store) store_transposed(a.dv + pr.qkv_off + li * a.s_l, db, g, acc);
  }
}

// ---------------------------------------------------------------------------------------------
// Any sequence length: the same one-wavefront-per-tile pieces in a loop over 32-key (or 32-query) blocks with a
// running softmax, so the [L, L] probabilities never go to memory.  Forward keeps log-sum-exp per query; backward
// recomputes the probabilities from it, once in a pass that owns a query block (dQ, and the row dot products
// delta = sum_d dO*O) and once in a pass that owns a key block (dK, dV): no atomics, fixed summation order.
// A wave works on its own LDS tiles and never meets another wave, so block counts may differ per wave (causal).
//
// The loops are bound by vector-ALU issue, not by the matrix cores (16 scores per lane and block against 8 MFMAs
// at D = 64), so the per-score work is kept to a handful of instructions: scores live in the log2 domain
// (scale * log2(e) folded into one FMA, the hardware 2^x), visibility tests only run in blocks that touch the
// end of the sequence or the causal diagonal, the running output is rescaled only when some query's maximum
// moved, and the loop-invariant operand fragments stay in registers.
struct FlashArgs {
  const bf16_t *q, *k, *v;
  bf16_t *dq, *dk, *dv;
  long s_l, s_b, s_h, s_g;  // element strides of q / k / v (and dq / dk / dv): sequence, batch, head, group
  bf16_t* o;                // forward output; backward reads it for delta
  const bf16_t* dout;
  long o_l, o_b, o_h, o_g;  // element strides of o / dout
  float* lse;               // [G*N*H][L] log-sum-exp of the scaled, masked scores
  float* delta;             // [G*N*H][L] row dot products dO . O (written by the dQ pass, read by the dK/dV pass)
  const float* mask;        // additive [L][L] or null
  const float* kbias;       // additive per (batch, key) [N][L] or null
  int causal;
  float scale;
  int L, N, H, nblk;  // nblk = ceil(L / 32)
  int nprob;          // G * N * H; nprob * nblk < 2^31
};

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// Orders a wave's LDS writes before its own later LDS reads of other lanes' data (no instruction is needed for
// that, the LDS serves a wave's accesses in order; this keeps the compiler from reordering them).
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

struct FlashItem {
  int z, blk, b;
  long qkv_off, o_off;
  bool live;
};
// `wave` is wave-uniform (scalar), so the whole item and every base address derived from it stay in scalar registers.
__device__ __forceinline__ FlashItem flash_locate(const FlashArgs& a, int wave, int waves_per_block) {
  FlashItem it;
  const unsigned total = (unsigned)a.nprob * (unsigned)a.nblk;
  unsigned w = blockIdx.x * (unsigned)waves_per_block + (unsigned)wave;
  it.live = w < total;
  if (!it.live) w = total - 1;  // idle waves redo the last item and store nothing
  // Block index major: with a causal mask the items of one block index are equally long, so the grid runs from the
  // longest items to the shortest, and the workgroups that share a CU (launch order modulo the CU count) differ in
  // length by whole strata instead of all being long or all being short.
  const unsigned blk = w / (unsigned)a.nprob, z = w - blk * (unsigned)a.nprob;
  it.z = (int)z;
  it.blk = (int)blk;
  const unsigned zh = z / (unsigned)a.H, h = z - zh * (unsigned)a.H;
  const unsigned g = zh / (unsigned)a.N, b = zh - g * (unsigned)a.N;
  it.qkv_off = (long)b * a.s_b + (long)h * a.s_h + (long)g * a.s_g;
  it.o_off = (long)b * a.o_b + (long)h * a.o_h + (long)g * a.o_g;
  it.b = (int)b;
  return it;
}

// NT tiles of one 32-row block, global -> registers -> LDS like TileRegs, for a loop: the lane's byte offsets inside
// a block are computed once (`prepare`), the block's base is a scalar, and rows beyond the sequence are redirected to
// row 0 only in the one ragged block.
template <int D, int NT>
struct BlockRegs {
  static constexpr int CPR = D / 8, NIT = kSeqMax * CPR / kWave;
  uint4 val[NT][NIT];
  unsigned ofs[NT][NIT];
  __device__ __forceinline__ void prepare(const long (&s_l)[NT], int lane) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + it * kWave, row = c / CPR, cc = c % CPR;
        ofs[t][it] = (unsigned)((row * s_l[t] + cc * 8) * (long)sizeof(bf16_t));
      }
  }
  __device__ __forceinline__ void fetch(const bf16_t* const (&base)[NT], int rows, int lane) {
    if (rows >= kSeqMax) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int it = 0; it < NIT; ++it)
          val[t][it] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(base[t]) + ofs[t][it]);
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
          const int c = lane + it * kWave, row = c / CPR, cc = c % CPR;
          const unsigned o = row < rows ? ofs[t][it] : (unsigned)(cc * 8 * sizeof(bf16_t));
          val[t][it] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(base[t]) + o);
        }
    }
  }
  __device__ __forceinline__ void commit(bf16_t* const (&tile)[NT], int rows, int lane) const {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int c = lane + it * kWave, row = c / CPR, cc = c % CPR;
        *reinterpret_cast<uint4*>(tile[t] + row * (D + 8) + cc * 8) = row < rows ? val[t][it] : make_uint4(0u, 0u, 0u, 0u);
      }
  }
};

// The 16 additive mask values of lane (li, g), times log2(e), for one query and the keys k0 + 8*(r/4) + 4*g + r%4
// (`keys_in_regs`), or for one key and the queries q0 + 8*(r/4) + 4*g + r%4: the [L][L] mask plus the per-(batch, key)
// bias.  Entries outside the sequence read element 0 (their scores are discarded anyway).
template <bool KEYS_IN_REGS>
__device__ __forceinline__ void flash_mask(const FlashArgs& a, int batch, int mine, int base, int g, float (&mk)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r) mk[r] = 0.0f;
  if (!a.mask && !a.kbias) return;
  if (a.mask) {
    if (KEYS_IN_REGS && a.L % 4 == 0 && reinterpret_cast<uintptr_t>(a.mask) % 16 == 0) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int key0 = base + 8 * a4 + 4 * g;
        const float4 m4 =
            *reinterpret_cast<const float4*>(a.mask + ((mine < a.L && key0 < a.L) ? (long)mine * a.L + key0 : 0));
        mk[4 * a4 + 0] = m4.x, mk[4 * a4 + 1] = m4.y, mk[4 * a4 + 2] = m4.z, mk[4 * a4 + 3] = m4.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int other = base + 8 * (r >> 2) + 4 * g + (r & 3);
        const long at = KEYS_IN_REGS ? (long)mine * a.L + other : (long)other * a.L + mine;
        mk[r] = a.mask[(mine < a.L && other < a.L) ? at : 0];
      }
    }
  }
  if (a.kbias) {
    const float* row = a.kbias + (long)batch * a.L;
    if (KEYS_IN_REGS) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = base + 8 * (r >> 2) + 4 * g + (r & 3);
        mk[r] += row[key < a.L ? key : 0];
      }
    } else {
      const float kb = row[mine < a.L ? mine : 0];
#pragma unroll
      for (int r = 0; r < 16; ++r) mk[r] += kb;
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) mk[r] *= kLog2e;
}

template <int D>
__device__ __forceinline__ void load_frags(const bf16_t* tile, int li, int g, bf16x8 (&f)[D / 16]) {
#pragma unroll
  for (int ks = 0; ks < D / 16; ++ks) f[ks] = frag_rowmajor(tile, D + 8, li, g, ks);
}

template <int DB, int NWV>
__global__ __launch_bounds__(NWV * 64) __attribute__((amdgpu_waves_per_eu(DB <= 2 ? 4 : 1))) void attn_flash_fwd_kernel(FlashArgs a) {
  touch_kernel_arguments<sizeof(FlashArgs)>();
  constexpr int D = 32 * DB, P = D + 8;
  constexpr bool PREFETCH = false;  // next block's K / V in registers while this one is worked on
  __shared__ __attribute__((aligned(16))) bf16_t tiles[NWV][2][kSeqMax * P];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const FlashItem it = flash_locate(a, wave, NWV);
  const int qb = a.nblk - 1 - it.blk;  // the long (causal) items first
  const int q0 = qb * kSeqMax, query = q0 + li;
  const bool qlive = query < a.L;
  bf16_t* Ks = tiles[wave][0];
  bf16_t* Vs = tiles[wave][1];
  const long kv_step = (long)kSeqMax * a.s_l;
  const bf16_t* kbase = a.k + it.qkv_off;
  const bf16_t* vbase = a.v + it.qkv_off;
  BlockRegs<D, 2> rkv;
  {
    const long sl2[2] = {a.s_l, a.s_l};
    rkv.prepare(sl2, lane);
  }
  bf16_t* const tl2[2] = {Ks, Vs};
  // the query block's fragments stay in registers; its tile only passes through the K tile's place
  bf16x8 qf[D / 16];
  {
    BlockRegs<D, 1> rq;
    const long sl[1] = {a.s_l};
    rq.prepare(sl, lane);
    const bf16_t* const src[1] = {a.q + it.qkv_off + (long)q0 * a.s_l};
    bf16_t* const tl[1] = {Ks};
    rq.fetch(src, a.L - q0, lane);
    rq.commit(tl, a.L - q0, lane);
    wave_sync();
    load_frags<D>(Ks, li, g, qf);
  }
  const int kb_end = a.causal ? qb : a.nblk - 1;
  if (PREFETCH) {
    const bf16_t* const src[2] = {kbase, vbase};
    rkv.fetch(src, a.L, lane);
  }
  const float scale2 = a.scale * kLog2e;
  float m_run = -INFINITY, l_run = 0.0f;  // running maximum (log2 domain) and sum
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.0f;
  for (int kb = 0; kb <= kb_end; ++kb) {
    const int k0 = kb * kSeqMax;
    if (!PREFETCH) {
      const bf16_t* const src[2] = {kbase + kb * kv_step, vbase + kb * kv_step};
      rkv.fetch(src, a.L - k0, lane);
    }
    wave_sync();  // the previous block's fragment reads are done
    rkv.commit(tl2, a.L - k0, lane);
    wave_sync();
    if (PREFETCH && kb < kb_end) {
      const bf16_t* const src[2] = {kbase + (kb + 1) * kv_step, vbase + (kb + 1) * kv_step};
      rkv.fetch(src, a.L - k0 - kSeqMax, lane);
    }
    float mk[16];
    flash_mask<true>(a, it.b, query, k0, g, mk);
    f32x16 s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Ks, P, li, g, ks), qf[ks], s, 0, 0, 0);
    float val[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) val[r] = fmaf(s[r], scale2, mk[r]);
    if (k0 + kSeqMax > a.L || (a.causal && kb == qb)) {  // wave-uniform: only these blocks hold hidden keys
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = k0 + 8 * (r >> 2) + 4 * g + (r & 3);
        const bool visible = key < a.L && (!a.causal || key <= query);
        val[r] = visible ? val[r] : -INFINITY;
      }
    }
    float bm = val[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) bm = fmaxf(bm, val[r]);
    bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
    const float m_new = fmaxf(m_run, bm);
    const float m_ref = m_new == -INFINITY ? 0.0f : m_new;  // everything hidden so far: 2^(-inf - 0) = 0 all round
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
    float rs = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      val[r] = __builtin_amdgcn_exp2f(val[r] - m_ref);
      rs += val[r];
    }
    rs += __shfl_xor(rs, 32, kWave);
    l_run = l_run * alpha + rs;
    m_run = m_new;
    bf16x8 pb[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) pb[r >> 3][r & 7] = from_f32<bf16_t>(val[r]);
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
    }
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int m = 0; m < 2; ++m)
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Vs, P, 32 * db, m, lane), pb[m], acc[db], 0,
                                                          0, 0);
  }
  const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
  if (it.live && qlive) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[db][r] *= inv;
      store_transposed(a.o + it.o_off + (long)query * a.o_l, db, g, acc[db]);
    }
    if (g == 0) a.lse[(long)it.z * a.L + query] = l_run > 0.0f ? (m_run + __builtin_amdgcn_logf(l_run)) * kLn2 : 0.0f;
  }
}

// Recomputed probabilities and score gradients of one (query block, key block) pair from the two accumulators
// s (scores) and dp: p[r] = 2^(scale2 * s + e[r]) with e = mask * log2(e) - lse * log2(e) prepared before the
// products, ds[r] = p * (scale * dp - sdelta) with sdelta = scale * delta per lane (KEYS_IN_REGS: the lane is a
// query) or per register (the lane is a key, registers run over queries).
template <bool KEYS_IN_REGS>
__device__ __forceinline__ void flash_p_ds(const FlashArgs& a, const f32x16& s, const f32x16& dp, const float (&e)[16],
                                           float scale2, int mine, int base, int g, bool edge,
                                           const float (&sdelta)[KEYS_IN_REGS ? 1 : 16], float (&pv)[16],
                                           float (&ds)[16]) {
#pragma unroll
  for (int r = 0; r < 16; ++r) pv[r] = __builtin_amdgcn_exp2f(fmaf(s[r], scale2, e[r]));
  if (edge) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int other = base + 8 * (r >> 2) + 4 * g + (r & 3);
      const int query = KEYS_IN_REGS ? mine : other, key = KEYS_IN_REGS ? other : mine;
      const bool visible = query < a.L && key < a.L && (!a.causal || key <= query);
      pv[r] = visible ? pv[r] : 0.0f;
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) ds[r] = pv[r] * fmaf(dp[r], a.scale, -sdelta[KEYS_IN_REGS ? 0 : r]);
}

template <int DB, int NWV>
__global__ __launch_bounds__(NWV * 64) __attribute__((amdgpu_waves_per_eu(DB <= 2 ? 3 : 1))) void attn_flash_dq_kernel(FlashArgs a) {
  touch_kernel_arguments<sizeof(FlashArgs)>();
  constexpr int D = 32 * DB, P = D + 8;
  constexpr bool PREFETCH = false;
  __shared__ __attribute__((aligned(16))) bf16_t tiles[NWV][2][kSeqMax * P];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const FlashItem it = flash_locate(a, wave, NWV);
  const int qb = a.nblk - 1 - it.blk;
  const int q0 = qb * kSeqMax, query = q0 + li;
  const bool qlive = query < a.L;
  bf16_t* Ks = tiles[wave][0];
  bf16_t* Vs = tiles[wave][1];
  const long kv_step = (long)kSeqMax * a.s_l;
  const bf16_t* kbase = a.k + it.qkv_off;
  const bf16_t* vbase = a.v + it.qkv_off;
  bf16_t* const tl2[2] = {Ks, Vs};
  // Q and dO fragments of the query block stay in registers; dO and O pass through the tiles for delta
  bf16x8 qf[D / 16], gf[D / 16];
  float delta = 0.0f;
  {
    BlockRegs<D, 2> rgo;
    const long sl[2] = {a.o_l, a.o_l};
    rgo.prepare(sl, lane);
    const bf16_t* const src[2] = {a.dout + it.o_off + (long)q0 * a.o_l, a.o + it.o_off + (long)q0 * a.o_l};
    rgo.fetch(src, a.L - q0, lane);
    rgo.commit(tl2, a.L - q0, lane);
    wave_sync();
    load_frags<D>(Ks, li, g, gf);
#pragma unroll
    for (int c = 0; c < D / 2; c += 8) {
      const bf16x8 gv = *reinterpret_cast<const bf16x8*>(Ks + li * P + g * (D / 2) + c);
      const bf16x8 ov = *reinterpret_cast<const bf16x8*>(Vs + li * P + g * (D / 2) + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) delta += to_f32(gv[e]) * to_f32(ov[e]);
    }
    delta += __shfl_xor(delta, 32, kWave);
    if (it.live && qlive && g == 0) a.delta[(long)it.z * a.L + query] = delta;
  }
  BlockRegs<D, 2> rkv;
  {
    const long sl2[2] = {a.s_l, a.s_l};
    rkv.prepare(sl2, lane);
    BlockRegs<D, 1> rq;
    const long sl[1] = {a.s_l};
    rq.prepare(sl, lane);
    const bf16_t* const src[1] = {a.q + it.qkv_off + (long)q0 * a.s_l};
    bf16_t* const tl[1] = {Ks};
    rq.fetch(src, a.L - q0, lane);
    wave_sync();  // the delta reads are done
    rq.commit(tl, a.L - q0, lane);
    wave_sync();
    load_frags<D>(Ks, li, g, qf);
  }
  const float lse2 = a.lse[(long)it.z * a.L + (qlive ? query : 0)] * kLog2e;
  const float sdelta[1] = {a.scale * delta};
  const int kb_end = a.causal ? qb : a.nblk - 1;
  if (PREFETCH) {
    const bf16_t* const src[2] = {kbase, vbase};
    rkv.fetch(src, a.L, lane);
  }
  const float scale2 = a.scale * kLog2e;
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.0f;
  for (int kb = 0; kb <= kb_end; ++kb) {
    const int k0 = kb * kSeqMax;
    if (!PREFETCH) {
      const bf16_t* const src[2] = {kbase + kb * kv_step, vbase + kb * kv_step};
      rkv.fetch(src, a.L - k0, lane);
    }
    wave_sync();
    rkv.commit(tl2, a.L - k0, lane);
    wave_sync();
    if (PREFETCH && kb < kb_end) {
      const bf16_t* const src[2] = {kbase + (kb + 1) * kv_step, vbase + (kb + 1) * kv_step};
      rkv.fetch(src, a.L - k0 - kSeqMax, lane);
    }
    float mk[16];
    flash_mask<true>(a, it.b, query, k0, g, mk);
#pragma unroll
    for (int r = 0; r < 16; ++r) mk[r] -= lse2;
    f32x16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Ks, P, li, g, ks), qf[ks], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Vs, P, li, g, ks), gf[ks], dp, 0, 0, 0);
    }
    const bool edge = q0 + kSeqMax > a.L || k0 + kSeqMax > a.L || (a.causal && kb == qb);
    float pv[16], ds[16];
    flash_p_ds<true>(a, s, dp, mk, scale2, query, k0, g, edge, sdelta, pv, ds);
    bf16x8 dsb[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) dsb[r >> 3][r & 7] = from_f32<bf16_t>(ds[r]);
    // dQ^T[dd][query] += sum_key K[key][dd] dS[query][key]
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int m = 0; m < 2; ++m)
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Ks, P, 32 * db, m, lane), dsb[m], acc[db], 0,
                                                          0, 0);
  }
  if (it.live && qlive) {
#pragma unroll
    for (int db = 0; db < DB; ++db) store_transposed(a.dq + it.qkv_off + (long)query * a.s_l, db, g, acc[db]);
  }
}

// Key-block pass.  Scores are formed as S[query][key] (A = Q rows, B = K rows), so a lane is a KEY and its 16
// accumulator registers run over the queries of the block: P and dS are then, as they stand, the B operands
// "lane = key, slots = queries" of dV^T = dO^T P and dK^T = Q^T dS, and the per-query statistics come in as 16
// values per lane.
template <int DB, int NWV>
__global__ __launch_bounds__(NWV * 64) __attribute__((amdgpu_waves_per_eu(DB <= 2 ? 2 : 1))) void attn_flash_dkv_kernel(FlashArgs a) {
  touch_kernel_arguments<sizeof(FlashArgs)>();
  constexpr int D = 32 * DB, P = D + 8;
  constexpr bool PREFETCH = DB <= 2;
  __shared__ __attribute__((aligned(16))) bf16_t tiles[NWV][2][kSeqMax * P];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, li = lane & 31, g = lane >> 5;
  const FlashItem it = flash_locate(a, wave, NWV);
  const int kb = it.blk;  // causal: key block 0 meets every query block, so the long items come first
  const int k0 = kb * kSeqMax, key = k0 + li;
  bf16_t* Qs = tiles[wave][0];
  bf16_t* Gs = tiles[wave][1];  // dO
  bf16_t* const tl2[2] = {Qs, Gs};
  // K and V fragments of the key block stay in registers; their tiles pass through the Q / dO tiles' place
  bf16x8 kf[D / 16], vf[D / 16];
  {
    BlockRegs<D, 2> rkv;
    const long sl[2] = {a.s_l, a.s_l};
    rkv.prepare(sl, lane);
    const bf16_t* const src[2] = {a.k + it.qkv_off + (long)k0 * a.s_l, a.v + it.qkv_off + (long)k0 * a.s_l};
    rkv.fetch(src, a.L - k0, lane);
    rkv.commit(tl2, a.L - k0, lane);
    wave_sync();
    load_frags<D>(Qs, li, g, kf);
    load_frags<D>(Gs, li, g, vf);
  }
  const int qb_start = a.causal ? kb : 0;
  const long q_step = (long)kSeqMax * a.s_l, g_step = (long)kSeqMax * a.o_l;
  const bf16_t* qbase = a.q + it.qkv_off;
  const bf16_t* gbase = a.dout + it.o_off;
  const float* lse_row = a.lse + (long)it.z * a.L;
  const float* delta_row = a.delta + (long)it.z * a.L;
  // queries come in runs of 4: with L % 4 == 0 whole runs are inside or outside the sequence (16-byte loads)
  const bool stat_quads = a.L % 4 == 0 && (reinterpret_cast<uintptr_t>(a.lse) | reinterpret_cast<uintptr_t>(a.delta)) % 16 == 0;
  BlockRegs<D, 2> rqg;
  {
    const long sl2[2] = {a.s_l, a.o_l};
    rqg.prepare(sl2, lane);
  }
  if (PREFETCH) {
    const bf16_t* const src[2] = {qbase + qb_start * q_step, gbase + qb_start * g_step};
    rqg.fetch(src, a.L - qb_start * kSeqMax, lane);
  }
  const float scale2 = a.scale * kLog2e;
  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) dk[db][r] = dv[db][r] = 0.0f;
  for (int qb = qb_start; qb < a.nblk; ++qb) {
    const int q0 = qb * kSeqMax;
    if (!PREFETCH) {
      const bf16_t* const src[2] = {qbase + qb * q_step, gbase + qb * g_step};
      rqg.fetch(src, a.L - q0, lane);
    }
    // statistics of the 16 queries of this lane's registers (the same for every key: broadcast loads)
    float lse_q[16], delta_q[16];
    if (stat_quads) {
#pragma unroll
      for (int a4 = 0; a4 < 4; ++a4) {
        const int query0 = q0 + 8 * a4 + 4 * g;
        const float4 l4 = *reinterpret_cast<const float4*>(lse_row + (query0 < a.L ? query0 : 0));
        const float4 d4 = *reinterpret_cast<const float4*>(delta_row + (query0 < a.L ? query0 : 0));
        lse_q[4 * a4 + 0] = l4.x, lse_q[4 * a4 + 1] = l4.y, lse_q[4 * a4 + 2] = l4.z, lse_q[4 * a4 + 3] = l4.w;
        delta_q[4 * a4 + 0] = d4.x, delta_q[4 * a4 + 1] = d4.y, delta_q[4 * a4 + 2] = d4.z, delta_q[4 * a4 + 3] = d4.w;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int query = q0 + 8 * (r >> 2) + 4 * g + (r & 3);
        lse_q[r] = lse_row[query < a.L ? query : 0];
        delta_q[r] = delta_row[query < a.L ? query : 0];
      }
    }
    wave_sync();  // the previous block's reads are done
    rqg.commit(tl2, a.L - q0, lane);
    wave_sync();
    if (PREFETCH && qb + 1 < a.nblk) {
      const bf16_t* const src[2] = {qbase + (qb + 1) * q_step, gbase + (qb + 1) * g_step};
      rqg.fetch(src, a.L - q0 - kSeqMax, lane);
    }
    float mk[16], sdelta[16];
    flash_mask<false>(a, it.b, key, q0, g, mk);
#pragma unroll
    for (int r = 0; r < 16; ++r) mk[r] = fmaf(lse_q[r], -kLog2e, mk[r]), sdelta[r] = delta_q[r] * a.scale;
    f32x16 s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = dp[r] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Qs, P, li, g, ks), kf[ks], s, 0, 0, 0);
      dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_rowmajor(Gs, P, li, g, ks), vf[ks], dp, 0, 0, 0);
    }
    const bool edge = q0 + kSeqMax > a.L || k0 + kSeqMax > a.L || (a.causal && kb == qb);
    float pv[16], ds[16];
    flash_p_ds<false>(a, s, dp, mk, scale2, key, q0, g, edge, sdelta, pv, ds);
    bf16x8 pb[2], dsb[2];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      pb[r >> 3][r & 7] = from_f32<bf16_t>(pv[r]);
      dsb[r >> 3][r & 7] = from_f32<bf16_t>(ds[r]);
    }
    // dK^T[dd][key] += sum_query Q[query][dd] dS[query][key];  dV^T[dd][key] += sum_query dO[query][dd] P[query][key]
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        dk[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Qs, P, 32 * db, m, lane), dsb[m], dk[db], 0, 0,
                                                         0);
        dv[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gather_acc_order(Gs, P, 32 * db, m, lane), pb[m], dv[db], 0, 0,
                                                         0);
      }
  }
  if (it.live && key < a.L) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      store_transposed(a.dk + it.qkv_off + (long)key * a.s_l, db, g, dk[db]);
      store_transposed(a.dv + it.qkv_off + (long)key * a.s_l, db, g, dv[db]);
    }
  }
}

static bool aligned8(int64_t v) { return v % 8 == 0; }

static int check_common(const char* who, int dtype, int64_t L, int64_t N, int64_t H, int64_t D, int64_t G, int64_t s_l,
                        int64_t s_b, int64_t s_h, int64_t s_g, int64_t o_l, int64_t o_b, int64_t o_h, int64_t o_g,
                        int64_t max_len = kSeqMax) {
  RTP_REQUIRE(dtype == RTP_BF16, "%s: only bf16 is implemented (dtype %d)", who, dtype);
  RTP_REQUIRE(L >= 1 && L <= max_len, "%s: sequence length %lld not in 1..%lld", who, (long long)L, (long long)max_len);
  RTP_REQUIRE(D == 32 || D == 64 || D == 128, "%s: head dimension %lld not in {32, 64, 128}", who, (long long)D);
  RTP_REQUIRE(N >= 1 && H >= 1 && G >= 1, "%s: batch, heads and groups must be >= 1", who);
  RTP_REQUIRE(aligned8(s_l) && aligned8(s_b) && aligned8(s_h) && aligned8(s_g) && aligned8(o_l) && aligned8(o_b) &&
                  aligned8(o_h) && aligned8(o_g),
              "%s: strides must be multiples of 8 elements", who);
  RTP_REQUIRE(G * N * H < (1ll << 31), "%s: too many problems", who);
  return RTP_OK;
}

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_attn_supported(int dtype, int64_t L, int64_t D) {
  return dtype == RTP_BF16 && L >= 1 && L <= kSeqMax && (D == 32 || D == 64 || D == 128);
}

extern "C" int rtp_attn_fwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                            int64_t s_b, int64_t s_h, int64_t s_g, void* o, int64_t o_l, int64_t o_b, int64_t o_h,
                            int64_t o_g, void* p, const float* mask, const float* key_bias, int causal, float scale,
                            int64_t L, int64_t N, int64_t H, int64_t D, int64_t G) {
  RTP_REQUIRE(q && k && v && o && p, "rtp_attn_fwd: null pointer");
  if (int rc = check_common("rtp_attn_fwd", dtype, L, N, H, D, G, s_l, s_b, s_h, s_g, o_l, o_b, o_h, o_g)) return rc;
  RTP_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) % 16 == 0,
              "rtp_attn_fwd: q, k, v, o must be 16-byte aligned");
  AttnArgs a{};
  a.q = (const bf16_t*)q, a.k = (const bf16_t*)k, a.v = (const bf16_t*)v;
  a.s_l = s_l, a.s_b = s_b, a.s_h = s_h, a.s_g = s_g;
  a.o = (bf16_t*)o, a.o_l = o_l, a.o_b = o_b, a.o_h = o_h, a.o_g = o_g;
  a.p = (bf16_t*)p, a.mask = mask, a.kbias = key_bias, a.causal = causal, a.scale = scale;
  a.L = (int)L, a.N = (int)N, a.H = (int)H, a.nprob = G * N * H;
  hipStream_t st = (hipStream_t)stream;
  const double np = (double)a.nprob;
  ProfileScope prof(st, "attn_fwd_small", 4.0 * np * L * L * D, np * (4.0 * L * D + (double)L * L) * 2.0);
  const unsigned grid = (unsigned)ceil_div(a.nprob, 4);
  if (D == 32)
    hipLaunchKernelGGL((attn_fwd_small_kernel<1, 4>), dim3(grid), dim3(256), 0, st, a);
  else if (D == 64)
    hipLaunchKernelGGL((attn_fwd_small_kernel<2, 4>), dim3(grid), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((attn_fwd_small_kernel<4, 4>), dim3(grid), dim3(256), 0, st, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_attn_bwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                            int64_t s_b, int64_t s_h, int64_t s_g, const void* dout, int64_t o_l, int64_t o_b,
                            int64_t o_h, int64_t o_g, const void* p, void* dq, void* dk, void* dv, float scale,
                            int64_t L, int64_t N, int64_t H, int64_t D, int64_t G) {
  RTP_REQUIRE(q && k && v && dout && p && dq && dk && dv, "rtp_attn_bwd: null pointer");
  if (int rc = check_common("rtp_attn_bwd", dtype, L, N, H, D, G, s_l, s_b, s_h, s_g, o_l, o_b, o_h, o_g)) return rc;
  RTP_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)dout | (uintptr_t)dq | (uintptr_t)dk |
               (uintptr_t)dv) % 16 == 0,
              "rtp_attn_bwd: q, k, v, dout, dq, dk, dv must be 16-byte aligned");
  AttnArgs a{};
  a.q = (const bf16_t*)q, a.k = (const bf16_t*)k, a.v = (const bf16_t*)v;
  a.dq = (bf16_t*)dq, a.dk = (bf16_t*)dk, a.dv = (bf16_t*)dv;
  a.s_l = s_l, a.s_b = s_b, a.s_h = s_h, a.s_g = s_g;
  a.dout = (const bf16_t*)dout, a.o_l = o_l, a.o_b = o_b, a.o_h = o_h, a.o_g = o_g;
  a.p = (bf16_t*)const_cast<void*>(p), a.scale = scale;
  a.L = (int)L, a.N = (int)N, a.H = (int)H, a.nprob = G * N * H;
  hipStream_t st = (hipStream_t)stream;
  const double np = (double)a.nprob;
  ProfileScope prof(st, "attn_bwd_small", 8.0 * np * L * L * D, np * (7.0 * L * D + (double)L * L) * 2.0);
  if (D == 32)
    hipLaunchKernelGGL((attn_bwd_small_kernel<1, 4>), dim3((unsigned)ceil_div(a.nprob, 4)), dim3(256), 0, st, a);
  else if (D == 64)
    hipLaunchKernelGGL((attn_bwd_small_kernel<2, 4>), dim3((unsigned)ceil_div(a.nprob, 4)), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((attn_bwd_small_kernel<4, 2>), dim3((unsigned)ceil_div(a.nprob, 2)), dim3(128), 0, st, a);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

// ---- any sequence length (running softmax over 32-key blocks) ----

static constexpr int64_t kFlashMaxLen = 1 << 20;

extern "C" int rtp_attn_flash_supported(int dtype, int64_t L, int64_t D) {
  return dtype == RTP_BF16 && L >= 1 && L <= kFlashMaxLen && (D == 32 || D == 64 || D == 128);
}

template <template <int, int> class Launcher>
static int flash_dispatch(int64_t D, const FlashArgs& a, hipStream_t st) {
  const long items = (long)a.nprob * a.nblk;
  if (D == 32)
    Launcher<1, 4>::run(a, st, items);
  else if (D == 64)
    Launcher<2, 4>::run(a, st, items);
  else
    Launcher<4, 2>::run(a, st, items);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
#define RTP_FLASH_LAUNCHER(NAME, KERNEL)                                                                       \
  template <int DB, int NWV>                                                                                   \
  struct NAME {                                                                                                \
    static void run(const FlashArgs& a, hipStream_t st, long items) {                                          \
      hipLaunchKernelGGL((KERNEL<DB, NWV>), dim3((unsigned)ceil_div(items, NWV)), dim3(NWV * 64), 0, st, a);   \
    }                                                                                                          \
  };
RTP_FLASH_LAUNCHER(FlashFwd, attn_flash_fwd_kernel)
RTP_FLASH_LAUNCHER(FlashDq, attn_flash_dq_kernel)
RTP_FLASH_LAUNCHER(FlashDkv, attn_flash_dkv_kernel)

static int flash_args(const char* who, FlashArgs& a, int dtype, int64_t s_l, int64_t s_b, int64_t s_h, int64_t s_g,
                      int64_t o_l, int64_t o_b, int64_t o_h, int64_t o_g, const float* mask, const float* key_bias,
                      int causal, float scale, int64_t L, int64_t N, int64_t H, int64_t D, int64_t G) {
  if (int rc = check_common(who, dtype, L, N, H, D, G, s_l, s_b, s_h, s_g, o_l, o_b, o_h, o_g, kFlashMaxLen)) return rc;
  a.s_l = s_l, a.s_b = s_b, a.s_h = s_h, a.s_g = s_g;
  a.o_l = o_l, a.o_b = o_b, a.o_h = o_h, a.o_g = o_g;
  a.mask = mask, a.kbias = key_bias, a.causal = causal, a.scale = scale;
  RTP_REQUIRE(G * N * H * ceil_div(L, kSeqMax) < (1ll << 31), "%s: too many (head, block) work items", who);
  // a lane's byte offsets inside one 32-row block are kept in 32 bits
  RTP_REQUIRE(s_l < (1ll << 25) && o_l < (1ll << 25) && s_l >= 0 && o_l >= 0, "%s: sequence stride out of range", who);
  a.L = (int)L, a.N = (int)N, a.H = (int)H, a.nblk = (int)ceil_div(L, kSeqMax), a.nprob = (int)(G * N * H);
  return RTP_OK;
}

extern "C" int rtp_attn_flash_fwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                                  int64_t s_b, int64_t s_h, int64_t s_g, void* o, int64_t o_l, int64_t o_b,
                                  int64_t o_h, int64_t o_g, float* lse, const float* mask, const float* key_bias,
                                  int causal, float scale, int64_t L, int64_t N, int64_t H, int64_t D, int64_t G) {
  RTP_REQUIRE(q && k && v && o && lse, "rtp_attn_flash_fwd: null pointer");
  RTP_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o) % 16 == 0,
              "rtp_attn_flash_fwd: q, k, v, o must be 16-byte aligned");
  FlashArgs a{};
  if (int rc = flash_args("rtp_attn_flash_fwd", a, dtype, s_l, s_b, s_h, s_g, o_l, o_b, o_h, o_g, mask, key_bias, causal,
                          scale, L, N, H, D, G))
    return rc;
  a.q = (const bf16_t*)q, a.k = (const bf16_t*)k, a.v = (const bf16_t*)v;
  a.o = (bf16_t*)o, a.lse = lse;
  hipStream_t st = (hipStream_t)stream;
  const double np = (double)a.nprob, vis = causal ? 0.5 : 1.0;
  ProfileScope prof(st, "attn_flash_fwd", 4.0 * np * L * L * D * vis, np * (4.0 * L * D * 2.0 + 4.0 * L));
  return flash_dispatch<FlashFwd>(D, a, st);
}

extern "C" int rtp_attn_flash_bwd(void* stream, int dtype, const void* q, const void* k, const void* v, int64_t s_l,
                                  int64_t s_b, int64_t s_h, int64_t s_g, const void* o, const void* dout, int64_t o_l,
                                  int64_t o_b, int64_t o_h, int64_t o_g, const float* lse, float* delta, void* dq,
                                  void* dk, void* dv, const float* mask, const float* key_bias, int causal, float scale,
                                  int64_t L, int64_t N, int64_t H, int64_t D, int64_t G) {
  RTP_REQUIRE(q && k && v && o && dout && lse && delta && dq && dk && dv, "rtp_attn_flash_bwd: null pointer");
  RTP_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)dout | (uintptr_t)dq |
               (uintptr_t)dk | (uintptr_t)dv) % 16 == 0,
              "rtp_attn_flash_bwd: q, k, v, o, dout, dq, dk, dv must be 16-byte aligned");
  FlashArgs a{};
  if (int rc = flash_args("rtp_attn_flash_bwd", a, dtype, s_l, s_b, s_h, s_g, o_l, o_b, o_h, o_g, mask, key_bias, causal,
                          scale, L, N, H, D, G))
    return rc;
  a.q = (const bf16_t*)q, a.k = (const bf16_t*)k, a.v = (const bf16_t*)v;
  a.dq = (bf16_t*)dq, a.dk = (bf16_t*)dk, a.dv = (bf16_t*)dv;
  a.o = (bf16_t*)const_cast<void*>(o), a.dout = (const bf16_t*)dout;
  a.lse = const_cast<float*>(lse), a.delta = delta;
  hipStream_t st = (hipStream_t)stream;
  const double np = (double)a.nprob, vis = causal ? 0.5 : 1.0;
  {
    // the query-block pass writes delta, the key-block pass reads it: same stream, in this order
    ProfileScope prof(st, "attn_flash_dq", 6.0 * np * L * L * D * vis, np * (5.0 * L * D * 2.0 + 8.0 * L));
    if (int rc = flash_dispatch<FlashDq>(D, a, st)) return rc;
  }
  ProfileScope prof(st, "attn_flash_dkv", 8.0 * np * L * L * D * vis, np * (6.0 * L * D * 2.0 + 8.0 * L));
  return flash_dispatch<FlashDkv>(D, a, st);
}
