// One rotated column-parallel Linear over ALL of its shards in one launch per product, the shards read straight
// from their home rows.  The loop the reference runs per layer (for every ring step: fetch the shard, multiply,
// concatenate -- rtp/module/linear.py:211-222, with its input gradient summed over the shards and its weight
// gradients written per shard in the backward, rtp/module/collectives.py:264-317) becomes a walk over
// (shard, tile) work items inside one product kernel: the loader waves stream the tiles of the next work item from
// home memory into the LDS stages while the MFMA waves work on the current one, so the LDS stage ring is the
// double buffer of the rotation and no second copy of a shard exists anywhere.
//
// Host code only: the three products are rtp_gemm launches with one group (forward, weight gradient) or one
// K segment (input gradient) per shard, visiting the shards in the ring order of rank 0.
#include "common.h"

#include <cstring>

using namespace rtp;

static int check_layer(const char* who, int dtype, const rtp_rotated_linear* L) {
  RTP_REQUIRE(L != nullptr && L->home != nullptr, "%s: null layer", who);
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "%s: unknown dtype %d", who, dtype);
  RTP_REQUIRE(L->shards >= 1 && L->n_s >= 1 && L->k >= 1 && L->w_off >= 0 && L->w_off + L->n_s * L->k <= L->numel,
              "%s: the weight [%lld, %lld] at offset %lld does not fit a flat shard of %lld elements", who,
              (long long)L->n_s, (long long)L->k, (long long)L->w_off, (long long)L->numel);
  RTP_REQUIRE(L->bias_off < 0 || L->bias_off + L->n_s <= L->numel, "%s: the bias does not fit the flat shard", who);
  return RTP_OK;
}

static void clear(rtp_gemm_desc* d) {
  memset(d, 0, sizeof(*d));
  d->batch = d->zdiv = d->groups = d->ksegs = 1;
  d->alpha = 1.0f;
}

extern "C" int rtp_rotated_linear_fwd(void* stream, int dtype, const rtp_rotated_linear* L, const void* x, int64_t ldx,
                                      int64_t rows, void* y, int64_t ldy, int flags) {
  if (int rc = check_layer("rtp_rotated_linear_fwd", dtype, L)) return rc;
  RTP_REQUIRE(x && y && ldx >= L->k && ldy >= L->n_s * L->shards, "rtp_rotated_linear_fwd: bad activations");
  RTP_REQUIRE((flags & ~(RTP_GEMM_RELU | RTP_GEMM_OUT_F32)) == 0, "rtp_rotated_linear_fwd: flags are RELU and OUT_F32");
  const int64_t es = dtype == RTP_F32 ? 4 : 2;
  rtp_gemm_desc d;
  clear(&d);
  d.a = x;
  d.b = (const char*)L->home + L->w_off * es;
  d.c_out = y;
  d.bias = L->bias_off >= 0 ? (const char*)L->home + L->bias_off * es : nullptr;
  d.m = rows, d.n = L->n_s, d.k = L->k;
  d.lda = ldx, d.ldb = L->k, d.ldc = ldy;
  d.groups = L->shards;
  d.b_sg = d.bias_sg = L->numel;  // shard g's flat buffer follows shard g-1's
  d.c_sg = L->n_s;                // its outputs are column block g
  d.flags = flags;
  d.a_kcontig = d.b_kcontig = 1;
  return rtp_gemm(stream, dtype, &d);
}

extern "C" int rtp_rotated_linear_bwd(void* stream, int dtype, const rtp_rotated_linear* L, const void* dy, int64_t ldy,
                                      const void* x, int64_t ldx, int64_t rows, const rtp_rotated_linear_bwd_args* o) {
  if (int rc = check_layer("rtp_rotated_linear_bwd", dtype, L)) return rc;
  RTP_REQUIRE(o != nullptr && dy && ldy >= L->n_s * L->shards, "rtp_rotated_linear_bwd: bad arguments");
  const int64_t es = dtype == RTP_F32 ? 4 : 2;
  if (o->dx) {
    // dX = (dx_init +) sum over the shards of dY[:, block g] W_g: one K segment per shard, summed in the accumulators
    RTP_REQUIRE(o->ld_dx >= L->k, "rtp_rotated_linear_bwd: ld_dx < k");
    rtp_gemm_desc d;
    clear(&d);
    d.a = dy;
    d.b = (const char*)L->home + L->w_off * es;
    d.c_out = o->dx;
    d.c_in = o->dx_init, d.ld_cin = o->ld_dx_init;
    d.gate = o->relu_gate, d.ld_gate = o->ld_relu_gate;
    RTP_REQUIRE((o->dx_flags & ~(int64_t)(RTP_GEMM_OUT_F32 | RTP_GEMM_CIN_F32)) == 0,
                "rtp_rotated_linear_bwd: dx_flags are OUT_F32 and CIN_F32");
    d.flags = (int32_t)o->dx_flags;
    d.m = rows, d.n = L->k, d.k = L->n_s;
    d.lda = ldy, d.ldb = L->k, d.ldc = o->ld_dx;
    d.ksegs = L->shards;
    d.a_sk = L->n_s, d.b_sk = L->numel;
    d.a_kcontig = 1, d.b_kcontig = 0;
    if (int rc = rtp_gemm(stream, dtype, &d)) return rc;
  }
  if (o->grads) {
    // dW_g = dY[:, block g]^T X into shard g's gradient row, the bias gradient (row sums of dY^T) from the same
    // launch where the kernel can carry it, and optionally the optimiser's update in the epilogue
    RTP_REQUIRE(x && ldx >= L->k, "rtp_rotated_linear_bwd: the weight gradient needs the layer's input");
    rtp_gemm_desc d;
    clear(&d);
    char* c = (char*)o->grads + L->w_off * es;
    d.a = dy;
    d.b = x;
    d.c_out = c;
    d.m = L->n_s, d.n = L->k, d.k = rows;
    d.lda = ldy, d.ldb = ldx, d.ldc = L->k;
    d.groups = L->shards;
    d.a_sg = L->n_s, d.c_sg = L->numel;
    if (o->accumulate) d.c_in = c, d.ld_cin = L->k, d.cin_sg = L->numel;
    d.flags = RTP_GEMM_STREAM_OUT | (o->accumulate ? RTP_GEMM_ROWSUM_ACCUM : 0);
    d.a_kcontig = d.b_kcontig = 0;
    const bool want_bias = L->bias_off >= 0;
    const bool bias_fused = want_bias && rtp_gemm_rowsum_fused(dtype, &d);
    if (bias_fused) d.a_rowsum = (char*)o->grads + L->bias_off * es, d.rowsum_sg = L->numel;
    int32_t done = 0;
    if (o->sgd_master) {
      RTP_REQUIRE(!o->accumulate, "rtp_rotated_linear_bwd: the fused update excludes gradient accumulation");
      const bool can = rtp_gemm_sgd_fused(dtype, &d) != 0;
      RTP_REQUIRE(can || o->done, "rtp_rotated_linear_bwd: these operands cannot take the fused update");
      if (can) {
        d.sgd_master = (char*)o->sgd_master + L->w_off * 4;
        d.sgd_weights = o->sgd_weights ? (char*)o->sgd_weights + L->w_off * es : nullptr;
        d.sgd_lr = o->sgd_lr, d.sgd_clip = o->sgd_clip;
        if (o->sgd_skip_grad_store) d.flags |= RTP_GEMM_SGD_SKIP_OUT;
        done |= RTP_ROTATED_SGD_DONE;
      }
    }
    if (int rc = rtp_gemm(stream, dtype, &d)) return rc;
    if (bias_fused) done |= RTP_ROTATED_BIAS_DONE;
    if (want_bias && !bias_fused) {
      const size_t need = rtp_colsum_workspace_bytes(rows, L->n_s * L->shards);
      if (o->colsum_workspace && o->colsum_workspace_bytes >= need) {
        if (int rc = rtp_colsum(stream, dtype, dy, rows, L->n_s * L->shards, ldy, (char*)o->grads + L->bias_off * es, 0,
                                o->accumulate, L->n_s, L->numel, o->colsum_workspace, o->colsum_workspace_bytes))
          return rc;
        done |= RTP_ROTATED_BIAS_DONE;
      } else {
        RTP_REQUIRE(o->done, "rtp_rotated_linear_bwd: the bias gradient of these operands needs a column-sum workspace of %zu bytes",
                    need);
      }
    }
    if (o->done) *o->done = done;
  } else if (o->done) {
    *o->done = 0;
  }
  return RTP_OK;
}

// ---- the logits layer together with its cross-entropy (rtp/models/transformer_lm_rtp.py:223 feeding the harness's
// nn.CrossEntropyLoss(), benchmarks/rtp_benchmark.py:182) -------------------------------------------------------
// Forward: the logits product leaves, per row, the softmax statistics of every 64-column block and the target's
// logit -- the [rows, classes] logits are never written -- and a small kernel turns them into the row's loss and
// {max, sum exp}.  Backward: the same product once more, its epilogue now writing the logits' gradient
// (softmax - onehot) * dloss * scale, which the layer's ordinary backward (rtp_rotated_linear_bwd) consumes.
static void logits_desc(rtp_gemm_desc* d, const rtp_rotated_linear* L, int64_t es, const void* x, int64_t ldx,
                        int64_t rows, void* out, int64_t ld_out) {
  clear(d);
  d->a = x;
  d->b = (const char*)L->home + L->w_off * es;
  d->c_out = out;
  d->bias = L->bias_off >= 0 ? (const char*)L->home + L->bias_off * es : nullptr;
  d->m = rows, d->n = L->n_s, d->k = L->k;
  d->lda = ldx, d->ldb = L->k, d->ldc = ld_out;
  d->groups = L->shards;
  d->b_sg = d->bias_sg = L->numel;
  d->c_sg = L->n_s;
  d->a_kcontig = d->b_kcontig = 1;
}

extern "C" size_t rtp_rotated_linear_xent_workspace_bytes(const rtp_rotated_linear* L, int64_t rows) {
  if (!L || rows <= 0 || L->n_s <= 0 || L->shards <= 0) return 256;
  return (size_t)rows * (size_t)(L->shards * L->n_s / 64) * 8 + (size_t)rows * 4 + 256;
}

extern "C" int rtp_rotated_linear_xent_fwd(void* stream, int dtype, const rtp_rotated_linear* L, const void* x,
                                           int64_t ldx, int64_t rows, const int64_t* target, int64_t ignore_index,
                                           float* loss, float* stats, void* workspace, size_t workspace_bytes) {
  if (int rc = check_layer("rtp_rotated_linear_xent_fwd", dtype, L)) return rc;
  RTP_REQUIRE(x && target && loss && stats && workspace && ldx >= L->k, "rtp_rotated_linear_xent_fwd: bad arguments");
  RTP_REQUIRE(L->n_s % 64 == 0, "rtp_rotated_linear_xent_fwd: a shard's %lld output columns are not a multiple of 64",
              (long long)L->n_s);
  RTP_REQUIRE((uintptr_t)workspace % 8 == 0 && workspace_bytes >= rtp_rotated_linear_xent_workspace_bytes(L, rows),
              "rtp_rotated_linear_xent_fwd: workspace of %zu bytes, need %zu (8-byte aligned)", workspace_bytes,
              rtp_rotated_linear_xent_workspace_bytes(L, rows));
  if (rows == 0) return RTP_OK;
  const int64_t es = dtype == RTP_F32 ? 4 : 2;
  const int64_t blocks = L->shards * L->n_s / 64;
  float* part = (float*)workspace;
  float* tlogit = part + rows * blocks * 2;
  rtp_gemm_desc d;
  // c_out is not written in this mode; the pointer only has to be a valid, aligned address for the descriptor checks
  logits_desc(&d, L, es, x, ldx, rows, workspace, L->n_s * L->shards);
  d.xent_mode = 1;
  d.xent_target = target, d.xent_ignore = ignore_index;
  d.xent_part = part, d.xent_tlogit = tlogit;
  if (int rc = rtp_gemm(stream, dtype, &d)) return rc;
  return rtp_softmax_xent_combine(stream, part, blocks, tlogit, target, ignore_index, rows, loss, stats);
}

extern "C" int rtp_rotated_linear_xent_bwd(void* stream, int dtype, const rtp_rotated_linear* L, const void* x,
                                           int64_t ldx, int64_t rows, const int64_t* target, int64_t ignore_index,
                                           const float* stats, const float* dloss, const float* scale, void* dlogits,
                                           int64_t ld_dlogits) {
  if (int rc = check_layer("rtp_rotated_linear_xent_bwd", dtype, L)) return rc;
  RTP_REQUIRE(x && target && stats && dloss && dlogits && ldx >= L->k && ld_dlogits >= L->n_s * L->shards,
              "rtp_rotated_linear_xent_bwd: bad arguments");
  RTP_REQUIRE(L->n_s % 64 == 0, "rtp_rotated_linear_xent_bwd: a shard's %lld output columns are not a multiple of 64",
              (long long)L->n_s);
  if (rows == 0) return RTP_OK;
  const int64_t es = dtype == RTP_F32 ? 4 : 2;
  rtp_gemm_desc d;
  logits_desc(&d, L, es, x, ldx, rows, dlogits, ld_dlogits);
  d.xent_mode = 2;
  d.xent_target = target, d.xent_ignore = ignore_index;
  d.xent_stats = stats, d.xent_dloss = dloss, d.xent_scale = scale;
  return rtp_gemm(stream, dtype, &d);
}
